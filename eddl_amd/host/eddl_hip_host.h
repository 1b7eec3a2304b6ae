// C++ host layer above the C ABI of libeddlhip.so.
//
// It mirrors, for the CNN forward path, the types and free functions that stand at EDDL's
// device-backend seam, with the reference's names, argument meaning and error behaviour, so
// that EDDL's Tensor / tensorNN dispatchers (or a program written against them) can call this
// backend where they call the CUDA one:
//   Tensor              include/eddl/tensor/tensor.h:72-103 (fields), src/tensor/tensor.cpp:107-263
//   ConvolDescriptor    include/eddl/descriptors/descriptors.h:67-157, src/descriptors/descriptor_conv2D.cpp
//   PoolDescriptor      include/eddl/descriptors/descriptors.h:426-481, src/descriptors/descriptor_pool2D.cpp
//   gpu_* functions     include/eddl/hardware/gpu/gpu_tensor.h:45-53, gpu_hw.h:30-257, nn/gpu_tensor_nn.h:26-147
//   tensorNN::*         src/tensor/nn/tensor_conv.cpp:30-66, tensor_pool.cpp:31-55,133-156,
//                       tensor_bn.cpp:93-129, tensor_activations.cpp:47-65,345-360,567-585
//   msg()               src/utils.cpp:57-67 (banner on stderr, then std::runtime_error("RuntimeError: " + title))
// Every gpu_* function here is synchronous on return, as the reference's wrappers are
// (they call cudaDeviceSynchronize after each launch, e.g. src/hardware/gpu/nn/gpu_pool.cu:27-33),
// unless gpu_set_synchronous(false) has been called: then compute calls return once queued on the
// device's stream, in order, and copies to the host still wait for everything queued before them.
// Everything lives in namespace eddl_hip so that it can be linked next to EDDL itself.
#pragma once
#include <string>
#include <vector>

namespace eddl_hip {

using std::string;
using std::vector;

constexpr int DEV_CPU = 0;
constexpr int DEV_GPU = 1000;  // DEV_GPU + i = GPU i, up to DEV_GPU_8 (tensor.h:28-53)

void msg(const string &text, const string &title = "");

class Tensor {
  public:
    int device;
    bool isshared = false;
    unsigned int ndim;
    unsigned long int size;
    vector<int> shape;
    vector<int> stride;
    float *ptr = nullptr;
    int gpu_device = -1;

    Tensor(const vector<int> &shape, int dev = DEV_CPU);               // allocates (host or device)
    Tensor(const vector<int> &shape, float *fptr, int dev = DEV_CPU);  // adopts fptr (host) or copies it to the device
    Tensor(const vector<int> &shape, Tensor *T);  // shares T's storage (isshared; src/tensor/tensor.cpp:78-79)
    void share(Tensor *T);                        // points a shared tensor at T's current storage again (T moved or resized)
    ~Tensor();
    Tensor(const Tensor &) = delete;
    Tensor &operator=(const Tensor &) = delete;

    bool isCPU() const { return device == DEV_CPU; }
    bool isGPU() const { return device >= DEV_GPU && device < 2000; }
    vector<int> getShape() const { return shape; }
    void updateStrides();
    void toGPU(int dev = DEV_GPU);
    void toCPU();
    void fill_(float v);
    // device-side initialisation (GPU tensors): src/tensor/tensor_generator.cpp:25-110, tensor_math.cpp:1455-1470
    void fill_rand_uniform_(float v);
    void fill_rand_signed_uniform_(float v);
    void fill_rand_normal_(float m, float s);
    void fill_rand_binary_(float v);
    void mult_(float v);
    void add_(float v);
    void resize(int b);                         // new batch size; storage is re-created
    void reshape_(const vector<int> &new_shape);  // same storage
    static Tensor *zeros(const vector<int> &shape, int dev = DEV_CPU);
    static Tensor *ones(const vector<int> &shape, int dev = DEV_CPU);
    static Tensor *full(const vector<int> &shape, float v, int dev = DEV_CPU);
    static void copy(Tensor *A, Tensor *B);  // any device pair
    // residual add / concat / resize / pad / dense, as the reference's static methods dispatch them
    static void add(float scA, Tensor *A, float scB, Tensor *B, Tensor *C, int incC);
    static void inc(Tensor *A, Tensor *B);
    static Tensor *concat(const vector<Tensor *> A, unsigned int axis = 0, Tensor *output = nullptr);
    static void scale(Tensor *A, Tensor *B, vector<int> new_shape, int wrapping_mode = 2, float cval = 0.0f,
                      int coordinate_transformation_mode = 3);
    static void pad(Tensor *A, Tensor *B, vector<int> pads);
    static void mult2D(Tensor *A, int tA, Tensor *B, int tB, Tensor *C, int incC);
    static void sum2D_rowwise(Tensor *A, Tensor *B, Tensor *C);

  private:
    void allocate();
    void release();
};

class ConvolDescriptor {
  public:
    vector<int> ksize, stride, pads;  // pads: {rows-top, rows-bottom, cols-left, cols-right}
    int nk, kr, kc, kz;
    int sr, sc;
    int in, ir, ic, iz;
    int r, c, z;
    int padrt, padrb, padcl, padcr;
    int filters;
    vector<int> kernel_size, strides;
    string padding;
    int groups;
    vector<int> dilation_rate;
    bool use_bias;
    int mem_level;
    Tensor *I = nullptr, *K = nullptr, *bias = nullptr, *O = nullptr;

    ConvolDescriptor(int filters, const vector<int> &kernel_size, const vector<int> &strides, string padding,
                     const vector<int> &pads, int groups, const vector<int> &dilation_rate, bool use_bias, int mem = 0);
    ~ConvolDescriptor();
    void build(Tensor *A);
    void resize(int b);
    static int compute_output(const string &padding, int input_size, int kernel_size, int stride, int dilation_rate = 1);
    static int compute_output(vector<int> padding, int input_size, int kernel_size, int stride, int dilation_rate = 1);
    static vector<int> compute_padding(int output_size, int input_size, int kernel_size, int stride, string padding = "same",
                                       bool row = false, int dilation_rate = 1);
};

class PoolDescriptor {
  public:
    vector<int> ksize, stride, pad;  // pad: {rows-top, rows-bottom, cols-left, cols-right}
    string padding;
    int kr, kc, sr, sc;
    int in, ir, ic, iz;
    int r, c, z;
    int padrt, padrb, padcl, padcr;
    int size;  // outputs per image the window walk writes
    int mem_level;
    Tensor *I = nullptr, *O = nullptr, *indX = nullptr, *indY = nullptr;

    PoolDescriptor(const vector<int> &ks, const vector<int> &st, const string &p, int mem = 0);
    PoolDescriptor(const vector<int> &ks, const vector<int> &st, const vector<int> &p, int mem = 0);
    ~PoolDescriptor();
    void build(Tensor *A);
    void resize(int b);
    static int compute_output(const string &padding, int input_size, int kernel_size, int stride, int dilation_rate = 1);
    static int compute_output(vector<int> padding, int input_size, int kernel_size, int stride, int dilation_rate = 1);
    static vector<int> compute_padding(int output_size, int input_size, int kernel_size, int stride, string padding = "same",
                                       bool row = false);
};

// ---- the backend seam: same signatures as the reference's gpu_* declarations.  They are defined, for this
// library and for EDDL itself, by one translation unit: integration/eddl/src/hardware/hip/hip_backend.cpp.
void gpu_init(int device);
void gpu_set_synchronous(bool on);      // no counterpart in the reference: see the note at the top
bool gpu_get_synchronous();
void gpu_synchronize(int gpu_device);   // waits for everything queued on the device
void gpu_check(int rc, const char *where);  // a C ABI return code -> the reference's exceptions
void gpu_set_random_seed(unsigned long long base);  // base seed of the device-side random fills (default 1234)
void gpu_delete_tensor_int(int dev, int *p);
void cpu2gpu(float *dst, const float *src, unsigned long int size, int gpu_device);
void gpu2cpu(float *dst, const float *src, unsigned long int size, int gpu_device);
float *get_gpu_fmem(unsigned long int size, int gpu_device);
void free_gpu_ptr(float *ptr, int gpu_device);
void gpu_rand_uniform(Tensor *A, float v);
void gpu_rand_signed_uniform(Tensor *A, float v);
void gpu_rand_binary(Tensor *A, float v);
void gpu_rand_normal(Tensor *A, float m, float s);
void gpu_mult(Tensor *A, Tensor *B, float v);
void gpu_add(Tensor *A, Tensor *B, float v);
void gpu_set_device(int device);
int gpu_devices();
float *gpu_create_tensor(int dev, int size);
void gpu_delete_tensor(int dev, float *p);
void gpu_copy_to_gpu(float *nptr, Tensor *B);
void gpu_copy_from_gpu(Tensor *A, float *nptr);
void gpu_copy_gpu(Tensor *A, Tensor *B);
void gpu_fill_(Tensor *A, float v);
void gpu_conv2D(ConvolDescriptor *D);
void gpu_mpool2D(PoolDescriptor *D);
void gpu_avgpool2D(PoolDescriptor *D);
void gpu_batchnorm_forward(int gpu_device, int b, int z, int rc, float *input, float *output, float *opa, float *global_mean,
                           float *global_variance, float *affine_g, float *affine_b, float *mean, float *variance, bool trmode,
                           float epsilon, float momentum);
void gpu_relu(Tensor *A, Tensor *B);
void gpu_sigmoid(Tensor *A, Tensor *B);
void gpu_full_softmax(Tensor *A, Tensor *B, int axis, bool stable);
void gpu_scale(Tensor *A, Tensor *B, vector<int> new_shape, int wrapping_mode, float constant, int transformation_mode);
void gpu_concat(Tensor *A, vector<Tensor *> t, unsigned int axis, bool derivative);
void gpu_add(float scA, Tensor *A, float scB, Tensor *B, Tensor *C, int incC);
void gpu_inc(Tensor *A, Tensor *B);
void gpu_pad(Tensor *A, Tensor *B, vector<int> pads);
void gpu_mult2D(Tensor *A, int tA, Tensor *B, int tB, Tensor *C, int incC);
void gpu_sum2D_rowwise(Tensor *A, Tensor *B, Tensor *C);

// ---- host wall-clock profile of the dispatchers, as the reference keeps it (include/eddl/profiling.h:27-66,
// src/profiling.cpp:200-330): per function, the number of calls and the microseconds between entry and return
// (gettimeofday).  With the wait after every gpu_* call the figure contains the kernel; with gpu_set_synchronous(false) it
// is the time to queue it.  Counter names are the reference's: forward, Conv2D, MPool2D, AvgPool2D, ReLu, Sigmoid,
// Softmax, add, inc, mult, mult2D, sum2D_rowwise, scale, fill_rand_uniform, fill_rand_signed_uniform, fill_rand_normal,
// fill_rand_binary.
struct ProfileCounter {
    const char *name;
    unsigned long long time_us = 0, calls = 0;
    explicit ProfileCounter(const char *n);
};
class ProfileScope {
  public:
    explicit ProfileScope(ProfileCounter &c);
    ~ProfileScope();

  private:
    ProfileCounter &counter;
    long long t0_us;
};
void __show_profile();   // the reference's two tables on stdout (src/profiling.cpp:200-330): "forward", then the functions called
void __reset_profile();  // src/profiling.cpp:332-480
ProfileCounter &profile_forward();  // the counter Net::forward charges (Net::do_forward, src/net/net_func.cpp:49-55)

// ---- the dispatchers the layers call (GPU branch only: this backend has no CPU path)
namespace tensorNN {
void Conv2D(ConvolDescriptor *D);
void MPool2D(PoolDescriptor *D);
void AvgPool2D(PoolDescriptor *D);
void BatchNormForward(Tensor *input, Tensor *output, Tensor *opa, Tensor *mean, Tensor *variance, Tensor *bn_g, Tensor *bn_b,
                      Tensor *bn_mean, Tensor *bn_var, bool trmode, float epsilon, float momentum);
void ReLu(Tensor *A, Tensor *B);
void Sigmoid(Tensor *A, Tensor *B);
void FullSoftmax(Tensor *A, Tensor *B, int axis, bool stable = true);
}  // namespace tensorNN

}  // namespace eddl_hip
