// The HIP binding of EDDL's device seam: definitions of the gpu_* functions that the CNN forward path, eddl::build
// and eddl::predict reach for a tensor on a GPU device, each one unpacking EDDL's objects into a call of
// libeddlhip.so's C ABI (include/eddlhip.h).  It replaces src/hardware/gpu/** in a build with -DcGPU -DcHIP;
// every other gpu_* declaration is defined in hip_stubs.cpp.
//
// The same text is compiled in two places:
//   inside EDDL          against EDDL's own headers: Tensor, ConvolDescriptor, PoolDescriptor are the real classes;
//   EDDLHIP_MIRROR_BUILD against eddl_hip_host.h of the backend's repository, whose classes carry the same member
//                        names (namespace eddl_hip): that build is what the backend's GPU tests run.
// Only members both have are used: Tensor::{gpu_device, ptr, size, ndim, shape, stride},
// ConvolDescriptor::{I, K, bias, O, use_bias, iz, ir, ic, nk, kr, kc, sr, sc, padrt, padcl, r, c},
// PoolDescriptor::{I, O, indX, indY, iz, ir, ic, kr, kc, sr, sc, padrt, padrb, padcl, padcr}.
#include <cstdlib>
#include <iostream>
#include <stdexcept>
#include <string>
#include <vector>

#ifdef EDDLHIP_MIRROR_BUILD
#include "eddl_hip_host.h"
#else
#include "eddl/descriptors/descriptors.h"
#include "eddl/hardware/gpu/gpu_hw.h"
#include "eddl/hardware/gpu/gpu_tensor.h"
#include "eddl/hardware/gpu/nn/gpu_tensor_nn.h"
#include "eddl/hardware/hip/hip_backend.h"
#include "eddl/tensor/tensor.h"
#include "eddl/utils.h"
#endif
#include "eddlhip.h"

#ifdef EDDLHIP_MIRROR_BUILD
namespace eddl_hip {
#endif

using std::string;
using std::vector;

// ---------------------------------------------------------------- errors and the wait after every call
void gpu_check(int rc, const char *where) {
    if (rc == 0) return;
    string text = eddlhip_last_error();
    if (rc == EDDLHIP_EINVAL) msg(text, where);
    throw std::runtime_error(string("[HIP ERROR]: ") + text + " (" + where + ")");
}

static bool hip_synchronous = true;

void gpu_set_synchronous(bool on) { hip_synchronous = on; }
bool gpu_get_synchronous() { return hip_synchronous; }
void gpu_synchronize(int gpu_device) { gpu_check(eddlhip_synchronize(gpu_device), "gpu_synchronize"); }

static void hip_done(int gpu_device) {
    if (hip_synchronous) gpu_synchronize(gpu_device);
}

// ---------------------------------------------------------------- runtime (gpu_tensor.h:45-53, gpu_hw.h:236-244)
static const int HIP_MAX_DEVICES = 16;
static bool hip_announced[HIP_MAX_DEVICES] = {false};

int gpu_devices() {
    int n = 0;
    gpu_check(eddlhip_device_count(&n), "gpu_devices");
    return n;
}

void gpu_init(int device) {
    int n = gpu_devices();
    if (device < 0 || device >= n || device >= HIP_MAX_DEVICES) {
        std::cerr << "[HIP ERROR]: GPU " << device << " not available. Number of available GPUs is " << n
                  << ". Further information running rocm-smi\n";
        throw std::runtime_error("[HIP ERROR]: device not available (gpu_init)");
    }
    gpu_check(eddlhip_init(device), "gpu_init");
    if (!hip_announced[device]) {
        char name[256];
        gpu_check(eddlhip_device_name(device, name, sizeof(name)), "gpu_init");
        std::cerr << "EDDL is running on GPU device " << device << ", " << name << "\n";
        hip_announced[device] = true;
        // The CUDA backend finds every convolution's algorithm by measurement on the layer's first forward
        // (cudnnFindConvolutionForwardAlgorithm, src/hardware/gpu/nn/gpu_conv.cu:42-66, 211-213).  The same here: the
        // library's plan search is on unless EDDLHIP_NO_TUNE is set, and EDDLHIP_PLANS=<file> starts it from the plans an
        // earlier process saved (eddlhip_conv2d_tuned_save), so that nothing is left to search for those geometries and
        // results are the same bits from run to run.
        const char *no_tune = getenv("EDDLHIP_NO_TUNE");
        if (no_tune == nullptr || no_tune[0] == 0 || no_tune[0] == '0') {
            const char *plans = getenv("EDDLHIP_PLANS");
            if (plans != nullptr && plans[0] != 0) gpu_check(eddlhip_conv2d_tuned_load(device, plans), "gpu_init (EDDLHIP_PLANS)");
            gpu_check(eddlhip_conv2d_autotune(1), "gpu_init");
        }
    }
}

void gpu_set_device(int device) { gpu_check(eddlhip_init(device), "gpu_set_device"); }

float *gpu_create_tensor(int dev, int size) {
    void *p = nullptr;
    gpu_check(eddlhip_malloc(dev, (size_t)size * sizeof(float), &p), "gpu_create_tensor");
    return (float *)p;
}

void gpu_delete_tensor(int dev, float *p) { gpu_check(eddlhip_free(dev, p), "gpu_delete_tensor"); }

void gpu_delete_tensor_int(int dev, int *p) { gpu_check(eddlhip_free(dev, p), "gpu_delete_tensor_int"); }

void gpu_copy_to_gpu(float *nptr, Tensor *B) {
    gpu_check(eddlhip_memcpy_h2d(B->gpu_device, B->ptr, nptr, B->size * sizeof(float)), "gpu_copy_to_gpu");
}

void gpu_copy_from_gpu(Tensor *A, float *nptr) {
    gpu_check(eddlhip_memcpy_d2h(A->gpu_device, nptr, A->ptr, A->size * sizeof(float)), "gpu_copy_from_gpu");
}

void gpu_copy_gpu(Tensor *A, Tensor *B) {
    gpu_check(eddlhip_memcpy_d2d(B->gpu_device, B->ptr, A->ptr, A->size * sizeof(float)), "gpu_copy_gpu");
    hip_done(B->gpu_device);
}

void cpu2gpu(float *dst, const float *src, unsigned long int size, int gpu_device) {
    gpu_check(eddlhip_memcpy_h2d(gpu_device, dst, src, size * sizeof(float)), "cpu2gpu");
}

void gpu2cpu(float *dst, const float *src, unsigned long int size, int gpu_device) {
    gpu_check(eddlhip_memcpy_d2h(gpu_device, dst, src, size * sizeof(float)), "gpu2cpu");
}

float *get_gpu_fmem(unsigned long int size, int gpu_device) {
    void *p = nullptr;
    gpu_check(eddlhip_malloc(gpu_device, size * sizeof(float), &p), "get_gpu_fmem");
    return (float *)p;
}

void free_gpu_ptr(float *ptr, int gpu_device) { gpu_check(eddlhip_free(gpu_device, ptr), "free_gpu_ptr"); }

void gpu_fill_(Tensor *A, float v) {
    gpu_check(eddlhip_fill(A->gpu_device, A->ptr, A->size, v), "gpu_fill_");
    hip_done(A->gpu_device);
}

// ---------------------------------------------------------------- parameter initialisation (gpu_hw.h:58-61,89,106)
// eddl::build initialises the device copy of a net on the device: Net::split -> make_graph -> do_initialize
// (src/net/net_build.cpp:235-237,401) -> e.g. IGlorotUniform::apply: fill_rand_signed_uniform_(1.0), mult_(limit).
static unsigned long long hip_seed_base = 1234;
static unsigned long long hip_fills[HIP_MAX_DEVICES] = {0};

void gpu_set_random_seed(unsigned long long base) {
    hip_seed_base = base;
    for (int i = 0; i < HIP_MAX_DEVICES; i++) hip_fills[i] = 0;
}

// one independent stream per fill: the base in the upper half of the generator's key, the fill's number in the lower
static unsigned long long hip_next_seed(int gpu_device) {
    const unsigned long long count = (gpu_device >= 0 && gpu_device < HIP_MAX_DEVICES) ? hip_fills[gpu_device]++ : 0;
    return (hip_seed_base << 32) ^ (count & 0xffffffffULL) ^ ((count >> 32) << 48);
}

void gpu_rand_uniform(Tensor *A, float v) {
    gpu_check(eddlhip_rand_uniform(A->gpu_device, A->ptr, A->size, v, hip_next_seed(A->gpu_device)), "gpu_rand_uniform");
    hip_done(A->gpu_device);
}

void gpu_rand_signed_uniform(Tensor *A, float v) {
    gpu_check(eddlhip_rand_signed_uniform(A->gpu_device, A->ptr, A->size, v, hip_next_seed(A->gpu_device)), "gpu_rand_signed_uniform");
    hip_done(A->gpu_device);
}

void gpu_rand_binary(Tensor *A, float v) {
    gpu_check(eddlhip_rand_binary(A->gpu_device, A->ptr, A->size, v, hip_next_seed(A->gpu_device)), "gpu_rand_binary");
    hip_done(A->gpu_device);
}

void gpu_rand_normal(Tensor *A, float m, float s) {
    gpu_check(eddlhip_rand_normal(A->gpu_device, A->ptr, A->size, m, s, hip_next_seed(A->gpu_device)), "gpu_rand_normal");
    hip_done(A->gpu_device);
}

void gpu_mult(Tensor *A, Tensor *B, float v) {
    gpu_check(eddlhip_mult_scalar(A->gpu_device, A->ptr, B->ptr, A->size, v), "gpu_mult");
    hip_done(A->gpu_device);
}

void gpu_add(Tensor *A, Tensor *B, float v) {
    gpu_check(eddlhip_add_scalar(A->gpu_device, A->ptr, B->ptr, A->size, v), "gpu_add");
    hip_done(A->gpu_device);
}

// ---------------------------------------------------------------- convolution and pooling (nn/gpu_tensor_nn.h:83,101,109)
void gpu_conv2D(ConvolDescriptor *D) {
    const int dev = D->I->gpu_device;
    gpu_check(eddlhip_conv2d_fwd(dev, D->I->ptr, D->K->ptr, D->use_bias ? D->bias->ptr : nullptr, D->O->ptr, D->I->shape[0], D->iz, D->ir,
                                 D->ic, D->nk, D->kr, D->kc, D->sr, D->sc, D->padrt, D->padcl, D->r, D->c, nullptr, nullptr, nullptr,
                                 nullptr, 0.0f, nullptr, 0),
              "gpu_conv2D");
    hip_done(dev);
}

// The window walk writes (rows visited) x (columns visited) outputs per plane; the descriptor's r x c output tensor
// must hold them (with the descriptors' own geometry it always does).
static void hip_check_pool_output(PoolDescriptor *D, const char *where) {
    int lp = 0, lq = 0;
    gpu_check(eddlhip_pool2d_out_dims(D->ir, D->ic, D->kr, D->kc, D->sr, D->sc, D->padrt, D->padrb, D->padcl, D->padcr, &lp, &lq), where);
    if ((unsigned long)D->I->shape[0] * D->iz * lp * lq > D->O->size) msg("the window walk writes more outputs than the output tensor holds", where);
}

void gpu_mpool2D(PoolDescriptor *D) {
    const int dev = D->I->gpu_device;
    hip_check_pool_output(D, "gpu_mpool2D");
    gpu_check(eddlhip_maxpool2d(dev, D->I->ptr, D->O->ptr, D->indX->ptr, D->indY->ptr, D->I->shape[0], D->iz, D->ir, D->ic, D->kr, D->kc,
                                D->sr, D->sc, D->padrt, D->padrb, D->padcl, D->padcr),
              "gpu_mpool2D");
    hip_done(dev);
}

void gpu_avgpool2D(PoolDescriptor *D) {
    const int dev = D->I->gpu_device;
    hip_check_pool_output(D, "gpu_avgpool2D");
    gpu_check(eddlhip_avgpool2d(dev, D->I->ptr, D->O->ptr, D->I->shape[0], D->iz, D->ir, D->ic, D->kr, D->kc, D->sr, D->sc, D->padrt,
                                D->padrb, D->padcl, D->padcr),
              "gpu_avgpool2D");
    hip_done(dev);
}

// ---------------------------------------------------------------- batch normalisation (nn/gpu_tensor_nn.h:138-143)
void gpu_batchnorm_forward(int gpu_device, int b, int z, int rc, float *input, float *output, float *opa, float *global_mean,
                           float *global_variance, float *affine_g, float *affine_b, float *mean, float *variance, bool trmode,
                           float epsilon, float momentum) {
    (void)mean;
    (void)momentum;
    if (trmode) msg("training-mode batch normalisation is outside this forward/inference backend", "gpu_batchnorm_forward");
    gpu_check(eddlhip_batchnorm_inference(gpu_device, b, z, rc, input, output, opa, global_mean, global_variance, affine_g, affine_b,
                                          variance, epsilon),
              "gpu_batchnorm_forward");
    hip_done(gpu_device);
}

// ---------------------------------------------------------------- activations (nn/gpu_tensor_nn.h:26,44,59)
void gpu_relu(Tensor *A, Tensor *B) {
    gpu_check(eddlhip_relu(A->gpu_device, A->ptr, B->ptr, A->size), "gpu_relu");
    hip_done(A->gpu_device);
}

void gpu_sigmoid(Tensor *A, Tensor *B) {
    gpu_check(eddlhip_sigmoid(A->gpu_device, A->ptr, B->ptr, A->size), "gpu_sigmoid");
    hip_done(A->gpu_device);
}

void gpu_full_softmax(Tensor *A, Tensor *B, int axis, bool stable) {
    int outer = 1, inner = 1;
    for (int i = 0; i < axis; i++) outer *= A->shape[i];
    for (unsigned i = axis + 1; i < A->ndim; i++) inner *= A->shape[i];
    gpu_check(eddlhip_softmax(A->gpu_device, A->ptr, B->ptr, outer, A->shape[axis], inner, stable ? 1 : 0), "gpu_full_softmax");
    hip_done(A->gpu_device);
}

// ---------------------------------------------------------------- resize, concat, add, pad (gpu_hw.h:46,66,71,112,113)
void gpu_scale(Tensor *A, Tensor *B, vector<int> new_shape, int wrapping_mode, float constant, int transformation_mode) {
    (void)constant;
    // UpSampling2D asks for nearest wrapping (2) and asymmetric coordinates (3): include/eddl/utils.h:119-122
    if (wrapping_mode != 2 || transformation_mode != 3)
        msg("only nearest wrapping with asymmetric coordinates is implemented on this backend", "gpu_scale");
    gpu_check(eddlhip_scale_nearest(A->gpu_device, A->ptr, B->ptr, A->shape[0], A->shape[1], A->shape[2], A->shape[3], B->shape[2],
                                    B->shape[3], new_shape[0], new_shape[1]),
              "gpu_scale");
    hip_done(A->gpu_device);
}

void gpu_concat(Tensor *A, vector<Tensor *> t, unsigned int axis, bool derivative) {
    if (derivative) msg("the backward of concat is outside this forward/inference backend", "gpu_concat");
    vector<const float *> srcs;
    vector<int> ext;
    for (Tensor *x : t) {
        srcs.push_back(x->ptr);
        ext.push_back(x->shape[axis]);
    }
    int outer = 1;
    for (unsigned i = 0; i < axis; i++) outer *= A->shape[i];
    gpu_check(eddlhip_concat(A->gpu_device, A->ptr, srcs.data(), ext.data(), (int)t.size(), outer, A->stride[axis]), "gpu_concat");
    hip_done(A->gpu_device);
}

void gpu_add(float scA, Tensor *A, float scB, Tensor *B, Tensor *C, int incC) {
    gpu_check(eddlhip_add(A->gpu_device, scA, A->ptr, scB, B->ptr, C->ptr, incC, A->size), "gpu_add");
    hip_done(A->gpu_device);
}

void gpu_inc(Tensor *A, Tensor *B) {
    gpu_check(eddlhip_inc(A->gpu_device, A->ptr, B->ptr, A->size), "gpu_inc");
    hip_done(A->gpu_device);
}

void gpu_pad(Tensor *A, Tensor *B, vector<int> pads) {
    gpu_check(eddlhip_pad(A->gpu_device, A->ptr, B->ptr, A->shape[0], A->shape[1], A->shape[2], A->shape[3], pads[0], pads[1], pads[2],
                          pads[3]),
              "gpu_pad");
    hip_done(A->gpu_device);
}

// ---------------------------------------------------------------- dense (gpu_hw.h:114,117)
void gpu_mult2D(Tensor *A, int tA, Tensor *B, int tB, Tensor *C, int incC) {
    if (tA || tB) msg("transposed operands belong to the backward pass, which is outside this backend", "gpu_mult2D");
    if (A->shape[1] != B->shape[0] || C->shape[0] != A->shape[0] || C->shape[1] != B->shape[1]) msg("Incompatible dims", "gpu_mult2D");
    gpu_check(eddlhip_mult2d(A->gpu_device, A->ptr, B->ptr, C->ptr, A->shape[0], A->shape[1], B->shape[1], incC), "gpu_mult2D");
    hip_done(A->gpu_device);
}

void gpu_sum2D_rowwise(Tensor *A, Tensor *B, Tensor *C) {
    gpu_check(eddlhip_sum2d_rowwise(A->gpu_device, A->ptr, B->ptr, C->ptr, A->shape[0], A->shape[1]), "gpu_sum2D_rowwise");
    hip_done(A->gpu_device);
}

#ifdef EDDLHIP_MIRROR_BUILD
}  // namespace eddl_hip
#endif
