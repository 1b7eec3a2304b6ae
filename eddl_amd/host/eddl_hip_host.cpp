// Implementation of the C++ host layer: reference-shaped objects unpacked into the flat
// C ABI of libeddlhip.so.  See eddl_hip_host.h for what each piece mirrors.
#include "eddl_hip_host.h"

#include <cmath>
#include <cstdlib>
#include <cstring>
#include <iostream>
#include <stdexcept>

#include <stdio.h>
#include <sys/time.h>

#include "../../include/eddlhip.h"

namespace eddl_hip {

// ---------------------------------------------------------------- errors
void msg(const string &text, const string &title) {
    string s(text);
    if (!title.empty()) s += " (" + title + ")";
    std::cerr << "==================================================================\n";
    std::cerr << "⚠️  " << s << " ⚠️" << std::endl;
    std::cerr << "==================================================================\n\n";
    throw std::runtime_error("RuntimeError: " + title);
}

// gpu_check, the wait after every call and every gpu_* function are defined in the binding translation unit,
// integration/eddl/src/hardware/hip/hip_backend.cpp, which the Makefile compiles into this library against the
// classes below (EDDLHIP_MIRROR_BUILD).

// ---------------------------------------------------------------- profile
static vector<ProfileCounter *> &profile_registry() {
    static vector<ProfileCounter *> all;
    return all;
}
ProfileCounter::ProfileCounter(const char *n) : name(n) { profile_registry().push_back(this); }

static long long now_us() {
    struct timeval tv;
    gettimeofday(&tv, nullptr);
    return (long long)tv.tv_sec * 1000000 + tv.tv_usec;
}
ProfileScope::ProfileScope(ProfileCounter &c) : counter(c), t0_us(now_us()) {}
ProfileScope::~ProfileScope() {
    counter.time_us += (unsigned long long)(now_us() - t0_us);
    counter.calls += 1;
}

#define EDDL_HIP_PROFILE(fn)                 \
    static ProfileCounter prof_##fn(#fn);    \
    ProfileScope prof_scope_##fn(prof_##fn)

ProfileCounter &profile_forward() {
    static ProfileCounter forward("forward");
    return forward;
}

static void profile_line(const ProfileCounter *c) {
    if (c->calls > 0)
        printf("| %-50s: %8lld calls, %12lld us , %12.4f us/call |\n", c->name, (long long)c->calls, (long long)c->time_us,
               (float)c->time_us / (float)c->calls);
}

void __show_profile() {
    const char *bar = "==============================================================================================================\n";
    const char *rule = "-------------------------------------------------------------------------------------------------------------|\n";
    printf("%s| Profiling (model)                                                                                          |\n%s", bar, rule);
    profile_line(&profile_forward());
    printf("%s| Profiling (functions)                                                                                      |\n%s", bar, rule);
    for (const ProfileCounter *c : profile_registry())
        if (c != &profile_forward()) profile_line(c);
    printf("%s", bar);
    fflush(stdout);
}

void __reset_profile() {
    profile_forward();
    for (ProfileCounter *c : profile_registry()) c->time_us = c->calls = 0;
}

// ---------------------------------------------------------------- Tensor
static void need_gpu(const Tensor *t, const char *where) {
    if (!t->isGPU()) msg("this backend only runs tensors that live on a GPU device", where);
}

void Tensor::updateStrides() {
    stride.assign(ndim, 1);
    for (int i = (int)ndim - 2; i >= 0; i--) stride[i] = stride[i + 1] * shape[i + 1];
}

void Tensor::allocate() {
    if (isCPU()) {
        void *p = nullptr;
        if (posix_memalign(&p, 64, (size ? size : 1) * sizeof(float)) != 0) msg("Error allocating memory", "Tensor::updateData");
        ptr = (float *)p;
    } else if (isGPU()) {
        gpu_device = device - DEV_GPU;
        gpu_init(gpu_device);  // once per device, on the first tensor (src/tensor/tensor.cpp:190-202)
        // gpu_create_tensor keeps the reference's signature, whose element count is an int
        if (size > 0x7fffffffUL) msg("A tensor of more than 2^31 - 1 elements does not fit gpu_create_tensor's int size", "Tensor::updateData");
        ptr = gpu_create_tensor(gpu_device, (int)size);
    } else {
        msg("Unsupported device", "Tensor::updateData");
    }
}

void Tensor::release() {
    if (ptr && !isshared) {
        if (isCPU()) free(ptr);
        else gpu_delete_tensor(gpu_device, ptr);
    }
    ptr = nullptr;
}

Tensor::Tensor(const vector<int> &shp, int dev) : device(dev), ndim((unsigned)shp.size()), shape(shp) {
    size = 1;
    for (int d : shape) size *= (unsigned long)d;
    updateStrides();
    allocate();
}

Tensor::Tensor(const vector<int> &shp, float *fptr, int dev) : device(dev), ndim((unsigned)shp.size()), shape(shp) {
    size = 1;
    for (int d : shape) size *= (unsigned long)d;
    updateStrides();
    if (isCPU()) {
        ptr = fptr;  // adopted, freed with the tensor
    } else {
        allocate();
        gpu_copy_to_gpu(fptr, this);
    }
}

Tensor::Tensor(const vector<int> &shp, Tensor *T) : device(T->device), isshared(true), ndim((unsigned)shp.size()), shape(shp) {
    size = 1;
    for (int d : shape) size *= (unsigned long)d;
    updateStrides();
    share(T);
}

void Tensor::share(Tensor *T) {
    if (!isshared) msg("only a tensor created as a view can be re-pointed", "Tensor::share");
    if (T->size != size) msg("Tensors with different size", "Tensor::share");
    device = T->device;
    gpu_device = T->gpu_device;
    ptr = T->ptr;
}

Tensor::~Tensor() { release(); }

void Tensor::toGPU(int dev) {
    if (!isCPU()) return;
    float *host = ptr;
    device = dev;
    ptr = nullptr;
    allocate();
    gpu_copy_to_gpu(host, this);
    free(host);
}

void Tensor::toCPU() {
    if (!isGPU()) return;
    void *p = nullptr;
    if (posix_memalign(&p, 64, (size ? size : 1) * sizeof(float)) != 0) msg("Error allocating memory", "Tensor::toCPU");
    gpu_copy_from_gpu(this, (float *)p);
    gpu_delete_tensor(gpu_device, ptr);
    ptr = (float *)p;
    device = DEV_CPU;
    gpu_device = -1;
}

void Tensor::fill_(float v) {
    if (isCPU()) {
        for (unsigned long i = 0; i < size; i++) ptr[i] = v;
    } else {
        gpu_fill_(this, v);
    }
}

// Random fills and scalar arithmetic as the reference's initialisers use them on a device tensor
// (src/tensor/tensor_generator.cpp:25-110, src/tensor/tensor_math.cpp:1455-1470)
void Tensor::fill_rand_uniform_(float v) {
    EDDL_HIP_PROFILE(fill_rand_uniform);
    need_gpu(this, "Tensor::fill_rand_uniform_");
    gpu_rand_uniform(this, v);
}
void Tensor::fill_rand_signed_uniform_(float v) {
    EDDL_HIP_PROFILE(fill_rand_signed_uniform);
    need_gpu(this, "Tensor::fill_rand_signed_uniform_");
    gpu_rand_signed_uniform(this, v);
}
void Tensor::fill_rand_normal_(float m, float s) {
    EDDL_HIP_PROFILE(fill_rand_normal);
    need_gpu(this, "Tensor::fill_rand_normal_");
    gpu_rand_normal(this, m, s);
}
void Tensor::fill_rand_binary_(float v) {
    EDDL_HIP_PROFILE(fill_rand_binary);
    need_gpu(this, "Tensor::fill_rand_binary_");
    gpu_rand_binary(this, v);
}
void Tensor::mult_(float v) {
    EDDL_HIP_PROFILE(mult);
    need_gpu(this, "Tensor::mult_");
    gpu_mult(this, this, v);
}
void Tensor::add_(float v) {
    EDDL_HIP_PROFILE(add);
    need_gpu(this, "Tensor::add_");
    gpu_add(this, this, v);
}

void Tensor::resize(int b) {
    if (b == shape[0]) return;
    release();
    shape[0] = b;
    size = 1;
    for (int d : shape) size *= (unsigned long)d;
    updateStrides();
    allocate();
}

void Tensor::reshape_(const vector<int> &new_shape) {
    unsigned long n = 1;
    for (int d : new_shape) n *= (unsigned long)d;
    if (n != size) msg("Not compatible shapes", "Tensor::reshape_");
    shape = new_shape;
    ndim = (unsigned)shape.size();
    updateStrides();
}

Tensor *Tensor::full(const vector<int> &shape, float v, int dev) {
    Tensor *t = new Tensor(shape, dev);
    t->fill_(v);
    return t;
}
Tensor *Tensor::zeros(const vector<int> &shape, int dev) { return full(shape, 0.0f, dev); }
Tensor *Tensor::ones(const vector<int> &shape, int dev) { return full(shape, 1.0f, dev); }

void Tensor::copy(Tensor *A, Tensor *B) {
    if (A->size != B->size) msg("Tensors with different size", "Tensor::copy");
    if (A->isCPU() && B->isCPU()) memcpy(B->ptr, A->ptr, A->size * sizeof(float));
    else if (A->isCPU() && B->isGPU()) gpu_copy_to_gpu(A->ptr, B);
    else if (A->isGPU() && B->isCPU()) gpu_copy_from_gpu(A, B->ptr);
    else gpu_copy_gpu(A, B);
}

void Tensor::add(float scA, Tensor *A, float scB, Tensor *B, Tensor *C, int incC) {
    EDDL_HIP_PROFILE(add);
    if (A->device != B->device || A->device != C->device) msg("Tensors in different devices", "Tensor::add");
    if (A->size != B->size || A->size != C->size) msg("Incompatible dims", "Tensor::add");
    need_gpu(A, "Tensor::add");
    gpu_add(scA, A, scB, B, C, incC);
}

void Tensor::inc(Tensor *A, Tensor *B) {
    EDDL_HIP_PROFILE(inc);
    if (A->size != B->size) msg("Tensors with different shape", "Tensor::inc");
    need_gpu(A, "Tensor::inc");
    gpu_inc(A, B);
}

Tensor *Tensor::concat(const vector<Tensor *> A, unsigned int axis, Tensor *output) {
    if (A.size() < 2) msg("Concat requires a minimum of two tensors", "Tensor::concat");
    vector<int> new_shape = A[0]->shape;
    int new_axis = 0;
    for (size_t i = 1; i < A.size(); i++) {
        if (A[0]->device != A[i]->device) msg("All tensors must be on the same device", "Tensor::concat");
        if (A[0]->ndim != A[i]->ndim) msg("The number of dimensions of all tensors must match", "Tensor::concat");
        for (size_t j = 0; j < A[0]->shape.size(); j++)
            if (j != axis && A[0]->shape[j] != A[i]->shape[j]) msg("The dimensions across of all tensors must match", "Tensor::concat");
        new_axis += A[i]->shape[axis];
    }
    new_shape[axis] += new_axis;
    if (output == nullptr) output = new Tensor(new_shape, A[0]->device);
    else if (output->shape != new_shape) msg("The dimension of the output tensor is incorrect", "Tensor::concat");
    else if (output->device != A[0]->device) msg("The output tensor and the input ones must be on the same device", "Tensor::concat");
    need_gpu(output, "Tensor::concat");
    gpu_concat(output, A, axis, false);
    return output;
}

void Tensor::scale(Tensor *A, Tensor *B, vector<int> new_shape, int wrapping_mode, float cval, int mode) {
    EDDL_HIP_PROFILE(scale);
    if (new_shape[0] <= 0 || new_shape[1] <= 0) msg("The new shape must be a greater than zero", "Tensor::scale");
    if (A->ndim != 4 || B->ndim != 4) msg("This method requires two 4D tensors", "Tensor::scale");
    if (A->device != B->device) msg("Tensors in different devices", "Tensor::scale");
    need_gpu(A, "Tensor::scale");
    gpu_scale(A, B, new_shape, wrapping_mode, cval, mode);
}

void Tensor::pad(Tensor *A, Tensor *B, vector<int> pads) {
    if (pads.size() == 2) pads = vector<int>({pads[0], pads[1], pads[0], pads[1]});
    else if (pads.size() != 4)
        msg("The padding on each border must follow this format (top-bottom, left-right) or (top, right, bottom, left)", "Tensor::pad");
    if (pads[0] < 0 || pads[1] < 0 || pads[2] < 0 || pads[3] < 0) msg("Pad margin must be greater or equal than zero", "Tensor::pad");
    if (A->ndim != 4 || B->ndim != 4) msg("This method requires two 4D tensors", "Tensor::pad");
    if (A->shape[0] != B->shape[0] || A->shape[1] != B->shape[1] || (A->shape[2] + (pads[0] + pads[2])) != B->shape[2] ||
        (A->shape[3] + (pads[1] + pads[3]) != B->shape[3]))
        msg("Incompatible dimensions", "Tensor::pad");
    if (A->device != B->device) msg("Tensors in different devices", "Tensor::pad");
    need_gpu(A, "Tensor::pad");
    gpu_pad(A, B, pads);
}

void Tensor::mult2D(Tensor *A, int tA, Tensor *B, int tB, Tensor *C, int incC) {
    EDDL_HIP_PROFILE(mult2D);
    if (A->device != B->device || A->device != C->device) msg("Tensors in different devices", "Tensor::mult2D");
    if (A->ndim != 2 || B->ndim != 2 || C->ndim != 2) msg("Only 2D tensors", "Tensor::mult2D");
    need_gpu(A, "Tensor::mult2D");
    gpu_mult2D(A, tA, B, tB, C, incC);
}

void Tensor::sum2D_rowwise(Tensor *A, Tensor *B, Tensor *C) {
    EDDL_HIP_PROFILE(sum2D_rowwise);
    if (A->ndim != 2 || B->ndim != 1 || C->ndim != 2) msg("sum2D_rowwise dims", "Tensor::sum2D_rowwise");
    if (A->shape[1] != B->shape[0] || A->shape != C->shape) msg("Incompatible dims", "Tensor::sum2D_rowwise");
    need_gpu(A, "Tensor::sum2D_rowwise");
    gpu_sum2D_rowwise(A, B, C);
}

// ---------------------------------------------------------------- window geometry, shared by both descriptors
// One routine holds the rules (float arithmetic as in the reference, src/descriptors/descriptor_conv2D.cpp:295-360,
// descriptor_pool2D.cpp:162-211): named paddings give out = ceil(in / stride) ("same", "zeros") or
// ceil((in - (k - 1) dilation) / stride) ("valid", "none") and the pads that go with it (total split low = pad / 2,
// high = the rest); "custom" takes the pads as given and out = int((in - (k - 1) dilation + lo + hi - 1) / stride + 1).
static int out_named(const string &padding, int input_size, int kernel_size, int stride, int dilation_rate, const char *where) {
    if (padding == "same" || padding == "zeros") return (int)std::ceil((float)input_size / (float)stride);
    if (padding == "valid" || padding == "none")
        return (int)std::ceil(((float)input_size - ((float)kernel_size - 1.0f) * (float)dilation_rate) / (float)stride);
    msg("Incorrect padding type", where);
    return -1;
}

static int out_custom(const vector<int> &padding, int input_size, int kernel_size, int stride, int dilation_rate) {
    return (int)(((float)input_size - ((float)kernel_size - 1.0f) * (float)dilation_rate + (float)padding[0] + (float)padding[1] - 1.0f) /
                     (float)stride +
                 1.0f);
}

static vector<int> pads_named(int output_size, int input_size, int kernel_size, int stride, string padding, bool row, int dilation_rate,
                              const char *where) {
    if (padding == "same,none") padding = row ? "same" : "none";
    if (padding == "none,same") padding = row ? "none" : "same";
    if (padding == "same" || padding == "zeros") {
        int pad = (output_size - 1) * stride + kernel_size - input_size + (dilation_rate - 1) * (kernel_size - 1);
        pad = std::max(pad, 0);
        return vector<int>({pad / 2, pad - pad / 2});
    }
    if (padding == "valid" || padding == "none") return vector<int>({0, 0});
    msg("Incorrect padding type", where);
    return {-1};
}

struct WindowGeometry {
    int r, c;          // output rows, columns
    vector<int> pads;  // {rows-top, rows-bottom, cols-left, cols-right}
};

// custom_cols_read_row_pads: PoolDescriptor::build hands the whole 4-vector to compute_output for both axes, which
// reads entries [0] and [1] (src/descriptors/descriptor_pool2D.cpp:78-79); ConvolDescriptor::build hands {pads[2], pads[3]}.
static WindowGeometry window_geometry(const char *who, const Tensor *A, const string &padding, const vector<int> &pads, int kr, int kc,
                                      int sr, int sc, int dil_r, int dil_c, bool custom_cols_read_row_pads) {
    const string where = string(who) + "::build";
    if (A->ndim != 4) msg("Tensors are not 4D", where);
    // (the reference reads these without a check; a graph from a file can hold anything)
    if (kr < 1 || kc < 1 || sr < 1 || sc < 1 || dil_r < 1 || dil_c < 1) msg("Kernel sizes, strides and dilations must be positive", where);
    if (padding == "custom" && pads.size() != 4) msg("Custom padding takes four values (top, bottom, left, right), got " + std::to_string(pads.size()), where);
    const int ir = A->shape[2], ic = A->shape[3];
    WindowGeometry g;
    if (padding == "custom") {
        g.pads = pads;
        g.r = out_custom({pads[0], pads[1]}, ir, kr, sr, dil_r);
        g.c = custom_cols_read_row_pads ? out_custom({pads[0], pads[1]}, ic, kc, sc, dil_c) : out_custom({pads[2], pads[3]}, ic, kc, sc, dil_c);
    } else {
        const string pr = padding == "same,none" ? "same" : padding == "none,same" ? "none" : padding;
        const string pc = padding == "same,none" ? "none" : padding == "none,same" ? "same" : padding;
        const string wo = string(who) + "::compute_output", wp = string(who) + "::compute_padding";
        g.r = out_named(pr, ir, kr, sr, dil_r, wo.c_str());
        g.c = out_named(pc, ic, kc, sc, dil_c, wo.c_str());
        const vector<int> padr = pads_named(g.r, ir, kr, sr, padding, true, dil_r, wp.c_str());
        const vector<int> padc = pads_named(g.c, ic, kc, sc, padding, false, dil_c, wp.c_str());
        g.pads = {padr[0], padr[1], padc[0], padc[1]};
    }
    if (g.r <= 0 || g.c <= 0) {
        if (g.r <= 0) std::cerr << "'Rows' are reach 0 or less (" << g.r << ")" << std::endl;
        if (g.c <= 0) std::cerr << "'Columns' are reach 0 or less (" << g.c << ")" << std::endl;
        msg("Invalid output shape", where);
    }
    return g;
}

// ---------------------------------------------------------------- ConvolDescriptor
ConvolDescriptor::ConvolDescriptor(int filters, const vector<int> &kernel_size, const vector<int> &strides, string padding,
                                   const vector<int> &pads, int groups, const vector<int> &dilation_rate, bool use_bias, int mem)
    : ksize(kernel_size), stride(strides), pads(pads), filters(filters), kernel_size(kernel_size), strides(strides), padding(padding),
      groups(groups), dilation_rate(dilation_rate), use_bias(use_bias), mem_level(mem) {
    const char *where = "ConvolDescriptor::ConvolDescriptor";
    if (groups > 1) msg("Grouped convolutions are only available with CuDNN", where);
    if (kernel_size.size() != 2) msg("Kernels must have 3 dimensions", where);
    if (strides.size() != 2) msg("Strides must have 2 dimensions", where);
    if (dilation_rate.size() != 2) msg("Dilations must have 2 elements", where);
    if (groups < 1) msg("The number of groups should be greater or equal to 1", where);
    ksize.insert(ksize.begin(), 1, filters);
    static const char *const known[] = {"custom", "same", "none", "valid", "zeros", "same,none", "none,same"};
    bool ok = false;
    for (const char *k : known) ok = ok || padding == k;
    if (!ok) msg("Incorrect padding type (" + padding + ")", where);
    if (filters % groups) msg("The number of filters must be divisible by the number groups.", where);
}

ConvolDescriptor::~ConvolDescriptor() {
    // O, K and bias belong to the layer that holds the descriptor (its output and params), as in the reference
}

int ConvolDescriptor::compute_output(const string &padding, int input_size, int kernel_size, int stride, int dilation_rate) {
    return out_named(padding, input_size, kernel_size, stride, dilation_rate, "ConvolDescriptor::compute_output");
}
int ConvolDescriptor::compute_output(vector<int> padding, int input_size, int kernel_size, int stride, int dilation_rate) {
    return out_custom(padding, input_size, kernel_size, stride, dilation_rate);
}
vector<int> ConvolDescriptor::compute_padding(int output_size, int input_size, int kernel_size, int stride, string padding, bool row,
                                              int dilation_rate) {
    return pads_named(output_size, input_size, kernel_size, stride, padding, row, dilation_rate, "ConvolDescriptor::compute_padding");
}

void ConvolDescriptor::build(Tensor *A) {
    const WindowGeometry g = window_geometry("ConvolDescriptor", A, padding, pads, ksize[1], ksize[2], stride[0], stride[1],
                                             dilation_rate[0], dilation_rate[1], false);
    if (A->shape[1] % groups) msg("The number of input channels must be divisible by the number groups.", "ConvolDescriptor::build");
    I = A;
    nk = z = ksize[0], kr = ksize[1], kc = ksize[2], kz = A->shape[1] / groups;
    sr = stride[0], sc = stride[1];
    in = A->shape[0], iz = A->shape[1], ir = A->shape[2], ic = A->shape[3];
    r = g.r, c = g.c, pads = g.pads;
    padrt = pads[0], padrb = pads[1], padcl = pads[2], padcr = pads[3];
    O = new Tensor(vector<int>{in, z, r, c}, A->device);
    K = new Tensor(vector<int>{nk, kz, kr, kc}, A->device);
    bias = new Tensor(vector<int>{nk}, A->device);
    // no lowering buffer: the convolution is an implicit GEMM
}

void ConvolDescriptor::resize(int b) {
    if (b == O->shape[0]) return;
    O->resize(b);
    in = b;
}

// ---------------------------------------------------------------- PoolDescriptor
PoolDescriptor::PoolDescriptor(const vector<int> &ks, const vector<int> &st, const vector<int> &p, int mem)
    : ksize(ks), stride(st), pad(p), padding("custom"), mem_level(mem) {
    if (ksize.size() != 2) msg("Pooling Kernels must have 2 dimensions", "PoolDescriptor::PoolDescriptor");
    if (stride.size() != 2) msg("Strides must have 2 dimensions", "PoolDescriptor::PoolDescriptor");
}

PoolDescriptor::PoolDescriptor(const vector<int> &ks, const vector<int> &st, const string &p, int mem)
    : ksize(ks), stride(st), padding(p), mem_level(mem) {
    if (ks.size() != 2) msg("Pooling Kernels must have 2 dimensions", "PoolDescriptor::PoolDescriptor");
    if (st.size() != 2) msg("Strides must have 2 dimensions", "PoolDescriptor::PoolDescriptor");
    if (!(p == "same" || p == "none" || p == "valid" || p == "zeros")) msg("Incorrect padding type", "PoolDescriptor::PoolDescriptor");
}

PoolDescriptor::~PoolDescriptor() {
    delete indX;
    delete indY;
}

int PoolDescriptor::compute_output(const string &padding, int input_size, int kernel_size, int stride, int dilation_rate) {
    return out_named(padding, input_size, kernel_size, stride, dilation_rate, "PoolDescriptor::compute_output");
}
int PoolDescriptor::compute_output(vector<int> padding, int input_size, int kernel_size, int stride, int dilation_rate) {
    return out_custom(padding, input_size, kernel_size, stride, dilation_rate);
}
vector<int> PoolDescriptor::compute_padding(int output_size, int input_size, int kernel_size, int stride, string padding, bool row) {
    return pads_named(output_size, input_size, kernel_size, stride, padding, row, 1, "PoolDescriptor::compute_padding");
}

void PoolDescriptor::build(Tensor *A) {
    const WindowGeometry g = window_geometry("PoolDescriptor", A, padding, pad, ksize[0], ksize[1], stride[0], stride[1], 1, 1, true);
    I = A;
    kr = ksize[0], kc = ksize[1], sr = stride[0], sc = stride[1];
    in = A->shape[0], iz = z = A->shape[1], ir = A->shape[2], ic = A->shape[3];
    r = g.r, c = g.c, pad = g.pads;
    padrt = pad[0], padrb = pad[1], padcl = pad[2], padcr = pad[3];
    O = new Tensor(vector<int>{in, z, r, c}, A->device);
    // outputs the window walk writes per image (the reference counts them by replaying its loop nest)
    const int rows = ir + padrb - kr >= -padrt ? (ir + padrb - kr + padrt) / sr + 1 : 0;
    const int cols = ic + padcr - kc >= -padcl ? (ic + padcr - kc + padcl) / sc + 1 : 0;
    size = iz * rows * cols;
}

void PoolDescriptor::resize(int b) {
    if (b == O->shape[0]) return;
    O->resize(b);
    in = b;
}

// ---------------------------------------------------------------- dispatchers
namespace tensorNN {

void Conv2D(ConvolDescriptor *D) {
    EDDL_HIP_PROFILE(Conv2D);
    if ((D->I->ndim != 4)) msg("Tensors are not 4D", "Tensor::Conv2D");
    if (D->dilation_rate[0] != 1 || D->dilation_rate[1] != 1) msg("Dilated convolutions are only available with CuDNN", "Tensor::Conv2D");
    need_gpu(D->I, "Tensor::Conv2D");
    gpu_conv2D(D);
}

void MPool2D(PoolDescriptor *D) {
    EDDL_HIP_PROFILE(MPool2D);
    if ((D->I->ndim != 4)) msg("Tensors are not 4D", "Tensor::MPool2D");
    need_gpu(D->I, "Tensor::MPool2D");
    gpu_mpool2D(D);
}

void AvgPool2D(PoolDescriptor *D) {
    EDDL_HIP_PROFILE(AvgPool2D);
    if ((D->I->ndim != 4)) msg("Tensors are not 4D", "Tensor::AvgPool2D");
    need_gpu(D->I, "Tensor::AvgPool2D");
    gpu_avgpool2D(D);
}

void BatchNormForward(Tensor *input, Tensor *output, Tensor *opa, Tensor *mean, Tensor *variance, Tensor *bn_g, Tensor *bn_b,
                      Tensor *bn_mean, Tensor *bn_var, bool trmode, float epsilon, float momentum) {
    need_gpu(input, "tensorNN::BatchNormForward");
    gpu_batchnorm_forward(input->gpu_device, input->shape[0], input->shape[1], input->ndim == 2 ? 1 : input->shape[2] * input->shape[3],
                          input->ptr, output->ptr, opa ? opa->ptr : nullptr, mean->ptr, variance->ptr, bn_g != NULL ? bn_g->ptr : NULL,
                          bn_b != NULL ? bn_b->ptr : NULL, bn_mean->ptr, bn_var->ptr, trmode, epsilon, momentum);
}

void ReLu(Tensor *A, Tensor *B) {
    EDDL_HIP_PROFILE(ReLu);
    if (A->device != B->device) msg("Tensors in different devices", "Tensor::ReLu");
    if (A->size != B->size) msg("Incompatible dims", "Tensor::ReLu");
    need_gpu(A, "Tensor::ReLu");
    gpu_relu(A, B);
}

void Sigmoid(Tensor *A, Tensor *B) {
    EDDL_HIP_PROFILE(Sigmoid);
    if (A->device != B->device) msg("Tensors in different devices", "Tensor::Sigmoid");
    if (A->size != B->size) msg("Incompatible dims", "Tensor::Sigmoid");
    need_gpu(A, "Tensor::Sigmoid");
    gpu_sigmoid(A, B);
}

void FullSoftmax(Tensor *A, Tensor *B, int axis, bool stable) {
    EDDL_HIP_PROFILE(Softmax);
    if (A->device != B->device) msg("Tensors in different devices", "Tensor::FullSoftmax");
    if (A->shape != B->shape) msg("Incompatible dims", "Tensor::FullSoftmax");
    need_gpu(A, "Tensor::FullSoftmax");
    gpu_full_softmax(A, B, axis, stable);
}

}  // namespace tensorNN
}  // namespace eddl_hip
