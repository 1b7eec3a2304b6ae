// Implementation of the C++ host layer: reference-shaped objects unpacked into the flat
// C ABI of libeddlhip.so.  See eddl_hip_host.h for what each piece mirrors.
#include "eddl_hip_host.h"

#include <cmath>
#include <cstdlib>
#include <cstring>
#include <iostream>
#include <stdexcept>

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

// A failed C ABI call becomes the reference's device-error exception
// (check_cuda throws std::runtime_error("[CUDA ERROR]: ..."), src/hardware/gpu/gpu_tensor.cu:103-112);
// a rejected argument becomes a msg().
void gpu_check(int rc, const char *where) {
    if (rc == 0) return;
    string text = eddlhip_last_error();
    if (rc == EDDLHIP_EINVAL) msg(text, where);
    throw std::runtime_error(string("[HIP ERROR]: ") + text + " (" + where + ")");
}

static void check(int rc, const char *where) { gpu_check(rc, where); }

static bool g_synchronous = true;

void gpu_set_synchronous(bool on) { g_synchronous = on; }
bool gpu_get_synchronous() { return g_synchronous; }
void gpu_synchronize(int gpu_device) { check(eddlhip_synchronize(gpu_device), "gpu_synchronize"); }

static void sync(int gpu_device) {
    if (g_synchronous) gpu_synchronize(gpu_device);
}

// ---------------------------------------------------------------- runtime
static bool g_init[16] = {false};

void gpu_init(int device) {
    int n = gpu_devices();
    if (device < 0 || device >= n) {
        std::cerr << "[HIP ERROR]: GPU " << device << " not available. Number of available GPUs is " << n
                  << ". Further information running rocm-smi\n";
        throw std::runtime_error("[HIP ERROR]: device not available (gpu_init)");
    }
    check(eddlhip_init(device), "gpu_init");
    if (!g_init[device]) {
        char name[256];
        check(eddlhip_device_name(device, name, sizeof(name)), "gpu_init");
        std::cerr << "EDDL is running on GPU device " << device << ", " << name << "\n";
        g_init[device] = true;
    }
}

void gpu_set_device(int device) { check(eddlhip_init(device), "gpu_set_device"); }

int gpu_devices() {
    int n = 0;
    check(eddlhip_device_count(&n), "gpu_devices");
    return n;
}

float *gpu_create_tensor(int dev, int size) {
    void *p = nullptr;
    check(eddlhip_malloc(dev, (size_t)size * sizeof(float), &p), "gpu_create_tensor");
    return (float *)p;
}

void gpu_delete_tensor(int dev, float *p) { check(eddlhip_free(dev, p), "gpu_delete_tensor"); }

void gpu_copy_to_gpu(float *nptr, Tensor *B) { check(eddlhip_memcpy_h2d(B->gpu_device, B->ptr, nptr, B->size * sizeof(float)), "gpu_copy_to_gpu"); }

void gpu_copy_from_gpu(Tensor *A, float *nptr) { check(eddlhip_memcpy_d2h(A->gpu_device, nptr, A->ptr, A->size * sizeof(float)), "gpu_copy_from_gpu"); }

void gpu_copy_gpu(Tensor *A, Tensor *B) {
    check(eddlhip_memcpy_d2d(B->gpu_device, B->ptr, A->ptr, A->size * sizeof(float)), "gpu_copy_gpu");
    sync(B->gpu_device);
}

void gpu_fill_(Tensor *A, float v) {
    check(eddlhip_fill(A->gpu_device, A->ptr, A->size, v), "gpu_fill_");
    sync(A->gpu_device);
}

// ---------------------------------------------------------------- Tensor
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

static void need_gpu(const Tensor *t, const char *where) {
    if (!t->isGPU()) msg("this backend only runs tensors that live on a GPU device", where);
}

void Tensor::add(float scA, Tensor *A, float scB, Tensor *B, Tensor *C, int incC) {
    if (A->device != B->device || A->device != C->device) msg("Tensors in different devices", "Tensor::add");
    if (A->size != B->size || A->size != C->size) msg("Incompatible dims", "Tensor::add");
    need_gpu(A, "Tensor::add");
    gpu_add(scA, A, scB, B, C, incC);
}

void Tensor::inc(Tensor *A, Tensor *B) {
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
    if (A->device != B->device || A->device != C->device) msg("Tensors in different devices", "Tensor::mult2D");
    if (A->ndim != 2 || B->ndim != 2 || C->ndim != 2) msg("Only 2D tensors", "Tensor::mult2D");
    need_gpu(A, "Tensor::mult2D");
    gpu_mult2D(A, tA, B, tB, C, incC);
}

void Tensor::sum2D_rowwise(Tensor *A, Tensor *B, Tensor *C) {
    if (A->ndim != 2 || B->ndim != 1 || C->ndim != 2) msg("sum2D_rowwise dims", "Tensor::sum2D_rowwise");
    if (A->shape[1] != B->shape[0] || A->shape != C->shape) msg("Incompatible dims", "Tensor::sum2D_rowwise");
    need_gpu(A, "Tensor::sum2D_rowwise");
    gpu_sum2D_rowwise(A, B, C);
}

// ---------------------------------------------------------------- geometry (float arithmetic as in the reference)
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

// ---------------------------------------------------------------- ConvolDescriptor
ConvolDescriptor::ConvolDescriptor(int filters, const vector<int> &kernel_size, const vector<int> &strides, string padding,
                                   const vector<int> &pads, int groups, const vector<int> &dilation_rate, bool use_bias, int mem) {
    const char *where = "ConvolDescriptor::ConvolDescriptor";
    if (groups > 1) msg("Grouped convolutions are only available with CuDNN", where);
    if (kernel_size.size() != 2) msg("Kernels must have 3 dimensions", where);
    if (strides.size() != 2) msg("Strides must have 2 dimensions", where);
    if (dilation_rate.size() != 2) msg("Dilations must have 2 elements", where);
    if (groups < 1) msg("The number of groups should be greater or equal to 1", where);
    this->filters = filters;
    this->kernel_size = kernel_size;
    this->strides = strides;
    this->padding = padding;
    this->pads = vector<int>(pads);
    this->groups = groups;
    this->dilation_rate = dilation_rate;
    this->use_bias = use_bias;
    this->mem_level = mem;
    ksize = vector<int>(kernel_size);
    ksize.insert(ksize.begin(), 1, filters);
    stride = vector<int>(strides);
    if (!(padding == "custom" || padding == "same" || padding == "none" || padding == "valid" || padding == "zeros" ||
          padding == "same,none" || padding == "none,same"))
        msg("Incorrect padding type (" + padding + ")", where);
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
    if (A->ndim != 4) msg("Tensors are not 4D", "ConvolDescriptor::build");
    I = A;
    nk = ksize[0];
    kr = ksize[1];
    kc = ksize[2];
    if (A->shape[1] % groups) msg("The number of input channels must be divisible by the number groups.", "ConvolDescriptor::build");
    kz = A->shape[1] / groups;
    sr = stride[0];
    sc = stride[1];
    in = A->shape[0];
    iz = A->shape[1];
    ir = A->shape[2];
    ic = A->shape[3];
    z = nk;
    if (padding == "custom") {
        r = compute_output(vector<int>{pads[0], pads[1]}, ir, kr, sr, dilation_rate[0]);
        c = compute_output(vector<int>{pads[2], pads[3]}, ic, kc, sc, dilation_rate[1]);
    } else {
        const string pr = padding == "same,none" ? "same" : padding == "none,same" ? "none" : padding;
        const string pc = padding == "same,none" ? "none" : padding == "none,same" ? "same" : padding;
        r = compute_output(pr, ir, kr, sr, dilation_rate[0]);
        c = compute_output(pc, ic, kc, sc, dilation_rate[1]);
        vector<int> padr = compute_padding(r, ir, kr, sr, padding, true, dilation_rate[0]);
        vector<int> padc = compute_padding(c, ic, kc, sc, padding, false, dilation_rate[1]);
        pads = {padr[0], padr[1], padc[0], padc[1]};
    }
    padrt = pads[0];
    padrb = pads[1];
    padcl = pads[2];
    padcr = pads[3];
    if (r <= 0 || c <= 0) {
        if (r <= 0) std::cerr << "'Rows' are reach 0 or less (" << r << ")" << std::endl;
        if (c <= 0) std::cerr << "'Columns' are reach 0 or less (" << c << ")" << std::endl;
        msg("Invalid output shape", "ConvolDescriptor::build");
    }
    O = new Tensor(vector<int>{A->shape[0], z, r, c}, A->device);
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
PoolDescriptor::PoolDescriptor(const vector<int> &ks, const vector<int> &st, const vector<int> &p, int mem) {
    ksize = ks;
    stride = st;
    pad = p;
    mem_level = mem;
    padding = "custom";
    if (ksize.size() != 2) msg("Pooling Kernels must have 2 dimensions", "PoolDescriptor::PoolDescriptor");
    if (stride.size() != 2) msg("Strides must have 2 dimensions", "PoolDescriptor::PoolDescriptor");
}

PoolDescriptor::PoolDescriptor(const vector<int> &ks, const vector<int> &st, const string &p, int mem) {
    if (ks.size() != 2) msg("Pooling Kernels must have 2 dimensions", "PoolDescriptor::PoolDescriptor");
    if (st.size() != 2) msg("Strides must have 2 dimensions", "PoolDescriptor::PoolDescriptor");
    ksize = ks;
    stride = st;
    mem_level = mem;
    if (p == "same" || p == "none" || p == "valid" || p == "zeros") padding = p;
    else msg("Incorrect padding type", "PoolDescriptor::PoolDescriptor");
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
    if (A->ndim != 4) msg("Tensors are not 4D", "PoolDescriptor::build");
    I = A;
    kr = ksize[0];
    kc = ksize[1];
    sr = stride[0];
    sc = stride[1];
    in = A->shape[0];
    iz = A->shape[1];
    ir = A->shape[2];
    ic = A->shape[3];
    z = iz;
    if (padding == "custom") {
        // as the reference: the whole 4-vector is handed over and entries [0], [1] are read for both axes
        r = compute_output(pad, ir, kr, sr);
        c = compute_output(pad, ic, kc, sc);
    } else {
        r = compute_output(padding, ir, kr, sr);
        c = compute_output(padding, ic, kc, sc);
        vector<int> padr = compute_padding(r, ir, kr, sr, padding, true);
        vector<int> padc = compute_padding(c, ic, kc, sc, padding, false);
        pad = {padr[0], padr[1], padc[0], padc[1]};
    }
    padrt = pad[0];
    padrb = pad[1];
    padcl = pad[2];
    padcr = pad[3];
    if (r <= 0 || c <= 0) {
        if (r <= 0) std::cerr << "'Rows' are reach 0 or less (" << r << ")" << std::endl;
        if (c <= 0) std::cerr << "'Columns' are reach 0 or less (" << c << ")" << std::endl;
        msg("Invalid output shape", "PoolDescriptor::build");
    }
    O = new Tensor(vector<int>{A->shape[0], z, r, c}, A->device);
    size = 0;
    for (int k = 0; k < iz; k++)
        for (int i = -padrt; i <= ir + padrb - kr; i += sr)
            for (int j = -padcl; j <= ic + padcr - kc; j += sc, size++) {
            }
}

void PoolDescriptor::resize(int b) {
    if (b == O->shape[0]) return;
    O->resize(b);
    in = b;
}

// ---------------------------------------------------------------- operators
void gpu_conv2D(ConvolDescriptor *D) {
    const int dev = D->I->gpu_device;
    check(eddlhip_conv2d_fwd(dev, D->I->ptr, D->K->ptr, D->use_bias ? D->bias->ptr : nullptr, D->O->ptr, D->I->shape[0], D->iz, D->ir,
                             D->ic, D->nk, D->kr, D->kc, D->sr, D->sc, D->padrt, D->padcl, D->r, D->c, nullptr, nullptr, nullptr, nullptr,
                             0.0f, nullptr, 0),
          "gpu_conv2D");
    sync(dev);
}

void gpu_mpool2D(PoolDescriptor *D) {
    const int dev = D->I->gpu_device;
    int lp = 0, lq = 0;
    check(eddlhip_pool2d_out_dims(D->ir, D->ic, D->kr, D->kc, D->sr, D->sc, D->padrt, D->padrb, D->padcl, D->padcr, &lp, &lq), "gpu_mpool2D");
    if ((unsigned long)D->I->shape[0] * D->iz * lp * lq > D->O->size) msg("the window walk writes more outputs than the output tensor holds", "gpu_mpool2D");
    check(eddlhip_maxpool2d(dev, D->I->ptr, D->O->ptr, D->indX->ptr, D->indY->ptr, D->I->shape[0], D->iz, D->ir, D->ic, D->kr, D->kc, D->sr,
                            D->sc, D->padrt, D->padrb, D->padcl, D->padcr),
          "gpu_mpool2D");
    sync(dev);
}

void gpu_avgpool2D(PoolDescriptor *D) {
    const int dev = D->I->gpu_device;
    int lp = 0, lq = 0;
    check(eddlhip_pool2d_out_dims(D->ir, D->ic, D->kr, D->kc, D->sr, D->sc, D->padrt, D->padrb, D->padcl, D->padcr, &lp, &lq), "gpu_avgpool2D");
    if ((unsigned long)D->I->shape[0] * D->iz * lp * lq > D->O->size) msg("the window walk writes more outputs than the output tensor holds", "gpu_avgpool2D");
    check(eddlhip_avgpool2d(dev, D->I->ptr, D->O->ptr, D->I->shape[0], D->iz, D->ir, D->ic, D->kr, D->kc, D->sr, D->sc, D->padrt, D->padrb,
                            D->padcl, D->padcr),
          "gpu_avgpool2D");
    sync(dev);
}

void gpu_batchnorm_forward(int gpu_device, int b, int z, int rc, float *input, float *output, float *opa, float *global_mean,
                           float *global_variance, float *affine_g, float *affine_b, float *mean, float *variance, bool trmode,
                           float epsilon, float momentum) {
    (void)mean;
    (void)momentum;
    if (trmode) msg("training-mode batch normalisation is outside this forward/inference backend", "gpu_batchnorm_forward");
    check(eddlhip_batchnorm_inference(gpu_device, b, z, rc, input, output, opa, global_mean, global_variance, affine_g, affine_b, variance,
                                      epsilon),
          "gpu_batchnorm_forward");
    sync(gpu_device);
}

void gpu_relu(Tensor *A, Tensor *B) {
    check(eddlhip_relu(A->gpu_device, A->ptr, B->ptr, A->size), "gpu_relu");
    sync(A->gpu_device);
}

void gpu_sigmoid(Tensor *A, Tensor *B) {
    check(eddlhip_sigmoid(A->gpu_device, A->ptr, B->ptr, A->size), "gpu_sigmoid");
    sync(A->gpu_device);
}

void gpu_full_softmax(Tensor *A, Tensor *B, int axis, bool stable) {
    int outer = 1, inner = 1;
    for (int i = 0; i < axis; i++) outer *= A->shape[i];
    for (unsigned i = axis + 1; i < A->ndim; i++) inner *= A->shape[i];
    check(eddlhip_softmax(A->gpu_device, A->ptr, B->ptr, outer, A->shape[axis], inner, stable ? 1 : 0), "gpu_full_softmax");
    sync(A->gpu_device);
}

void gpu_scale(Tensor *A, Tensor *B, vector<int> new_shape, int wrapping_mode, float constant, int transformation_mode) {
    (void)constant;
    // UpSampling2D asks for nearest wrapping (2) and asymmetric coordinates (3): include/eddl/utils.h:119-122
    if (wrapping_mode != 2 || transformation_mode != 3)
        msg("only nearest wrapping with asymmetric coordinates is implemented on this backend", "gpu_scale");
    check(eddlhip_scale_nearest(A->gpu_device, A->ptr, B->ptr, A->shape[0], A->shape[1], A->shape[2], A->shape[3], B->shape[2], B->shape[3],
                                new_shape[0], new_shape[1]),
          "gpu_scale");
    sync(A->gpu_device);
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
    check(eddlhip_concat(A->gpu_device, A->ptr, srcs.data(), ext.data(), (int)t.size(), outer, A->stride[axis]), "gpu_concat");
    sync(A->gpu_device);
}

void gpu_add(float scA, Tensor *A, float scB, Tensor *B, Tensor *C, int incC) {
    check(eddlhip_add(A->gpu_device, scA, A->ptr, scB, B->ptr, C->ptr, incC, A->size), "gpu_add");
    sync(A->gpu_device);
}

void gpu_inc(Tensor *A, Tensor *B) {
    check(eddlhip_inc(A->gpu_device, A->ptr, B->ptr, A->size), "gpu_inc");
    sync(A->gpu_device);
}

void gpu_pad(Tensor *A, Tensor *B, vector<int> pads) {
    check(eddlhip_pad(A->gpu_device, A->ptr, B->ptr, A->shape[0], A->shape[1], A->shape[2], A->shape[3], pads[0], pads[1], pads[2], pads[3]),
          "gpu_pad");
    sync(A->gpu_device);
}

void gpu_mult2D(Tensor *A, int tA, Tensor *B, int tB, Tensor *C, int incC) {
    if (tA || tB) msg("transposed operands belong to the backward pass, which is outside this backend", "gpu_mult2D");
    if (A->shape[1] != B->shape[0] || C->shape[0] != A->shape[0] || C->shape[1] != B->shape[1]) msg("Incompatible dims", "gpu_mult2D");
    check(eddlhip_mult2d(A->gpu_device, A->ptr, B->ptr, C->ptr, A->shape[0], A->shape[1], B->shape[1], incC), "gpu_mult2D");
    sync(A->gpu_device);
}

void gpu_sum2D_rowwise(Tensor *A, Tensor *B, Tensor *C) {
    check(eddlhip_sum2d_rowwise(A->gpu_device, A->ptr, B->ptr, C->ptr, A->shape[0], A->shape[1]), "gpu_sum2D_rowwise");
    sync(A->gpu_device);
}

// ---------------------------------------------------------------- dispatchers
namespace tensorNN {

void Conv2D(ConvolDescriptor *D) {
    if ((D->I->ndim != 4)) msg("Tensors are not 4D", "Tensor::Conv2D");
    if (D->dilation_rate[0] != 1 || D->dilation_rate[1] != 1) msg("Dilated convolutions are only available with CuDNN", "Tensor::Conv2D");
    need_gpu(D->I, "Tensor::Conv2D");
    gpu_conv2D(D);
}

void MPool2D(PoolDescriptor *D) {
    if ((D->I->ndim != 4)) msg("Tensors are not 4D", "Tensor::MPool2D");
    need_gpu(D->I, "Tensor::MPool2D");
    gpu_mpool2D(D);
}

void AvgPool2D(PoolDescriptor *D) {
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
    if (A->device != B->device) msg("Tensors in different devices", "Tensor::ReLu");
    if (A->size != B->size) msg("Incompatible dims", "Tensor::ReLu");
    need_gpu(A, "Tensor::ReLu");
    gpu_relu(A, B);
}

void Sigmoid(Tensor *A, Tensor *B) {
    if (A->device != B->device) msg("Tensors in different devices", "Tensor::Sigmoid");
    if (A->size != B->size) msg("Incompatible dims", "Tensor::Sigmoid");
    need_gpu(A, "Tensor::Sigmoid");
    gpu_sigmoid(A, B);
}

void FullSoftmax(Tensor *A, Tensor *B, int axis, bool stable) {
    if (A->device != B->device) msg("Tensors in different devices", "Tensor::FullSoftmax");
    if (A->shape != B->shape) msg("Incompatible dims", "Tensor::FullSoftmax");
    need_gpu(A, "Tensor::FullSoftmax");
    gpu_full_softmax(A, B, axis, stable);
}

}  // namespace tensorNN
}  // namespace eddl_hip
