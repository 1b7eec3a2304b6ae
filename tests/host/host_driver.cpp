// Descriptor-level driver of the C++ host layer, written the way the reference's own unit
// tests use the seam (new ConvolDescriptor -> build -> set K/bias -> tensorNN::Conv2D, as in
// tests/layers/conv/test_conv2d.cpp:109-123): the Python tests write the inputs as raw float32
// files, this program runs them through eddl_hip::{Tensor, *Descriptor, tensorNN::*} on GPU 0
// and writes the outputs back for comparison with the CPU oracle.
//
//   host_driver <case> <dir>      case = conv2d | mpool | avgpool | bn | chain | errors
#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <iostream>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

#include "eddl_hip_host.h"

using namespace eddl_hip;

static std::string g_dir;

static std::vector<std::string> read_params() {
    std::ifstream f(g_dir + "/params.txt");
    if (!f) throw std::runtime_error("cannot read params.txt");
    std::vector<std::string> v;
    std::string tok;
    while (f >> tok) v.push_back(tok);
    return v;
}

static float *read_bin(const std::string &name, size_t n) {
    float *p = nullptr;
    if (posix_memalign((void **)&p, 64, (n ? n : 1) * sizeof(float)) != 0) throw std::runtime_error("alloc");
    FILE *f = fopen((g_dir + "/" + name).c_str(), "rb");
    if (!f) throw std::runtime_error("cannot open " + name);
    if (fread(p, sizeof(float), n, f) != n) throw std::runtime_error("short read of " + name);
    fclose(f);
    return p;
}

static void write_tensor(const std::string &name, Tensor *t) {
    t->toCPU();
    FILE *f = fopen((g_dir + "/" + name + ".bin").c_str(), "wb");
    fwrite(t->ptr, sizeof(float), t->size, f);
    fclose(f);
    std::ofstream s(g_dir + "/" + name + ".shape");
    for (int d : t->shape) s << d << " ";
}

static Tensor *gpu_tensor(const std::vector<int> &shape, const std::string &file) {
    size_t n = 1;
    for (int d : shape) n *= d;
    Tensor *t = new Tensor(shape, read_bin(file, n), DEV_CPU);
    t->toGPU(DEV_GPU);
    return t;
}

static std::vector<int> ints(const std::vector<std::string> &p, size_t from, size_t count) {
    std::vector<int> v;
    for (size_t i = 0; i < count; i++) v.push_back(atoi(p[from + i].c_str()));
    return v;
}

static int run_conv2d() {
    // params: N C H W filters kr kc sr sc use_bias padding [pt pb pl pr]
    auto p = read_params();
    auto s = ints(p, 0, 10);
    std::string padding = p[10];
    std::vector<int> pads = padding == "custom" ? ints(p, 11, 4) : std::vector<int>{};
    Tensor *t_image = gpu_tensor({s[0], s[1], s[2], s[3]}, "I.bin");
    auto *cd = new ConvolDescriptor(s[4], {s[5], s[6]}, {s[7], s[8]}, padding, pads, 1, {1, 1}, s[9] != 0);
    cd->build(t_image);
    delete cd->K;
    delete cd->bias;
    cd->K = gpu_tensor({s[4], s[1], s[5], s[6]}, "K.bin");
    cd->bias = gpu_tensor({s[4]}, "bias.bin");
    tensorNN::Conv2D(cd);
    write_tensor("O", cd->O);
    return 0;
}

static int run_pool(bool is_max) {
    // params: N C H W kr kc sr sc padding [pt pb pl pr]
    auto p = read_params();
    auto s = ints(p, 0, 8);
    std::string padding = p[8];
    Tensor *t_image = gpu_tensor({s[0], s[1], s[2], s[3]}, "I.bin");
    PoolDescriptor *pd = padding == "custom" ? new PoolDescriptor({s[4], s[5]}, {s[6], s[7]}, ints(p, 9, 4))
                                             : new PoolDescriptor({s[4], s[5]}, {s[6], s[7]}, padding);
    pd->build(t_image);
    if (is_max) {
        pd->indX = Tensor::full(pd->O->getShape(), -1.0f, pd->O->device);
        pd->indY = Tensor::full(pd->O->getShape(), -1.0f, pd->O->device);
        tensorNN::MPool2D(pd);
        write_tensor("indX", pd->indX);
        write_tensor("indY", pd->indY);
    } else {
        tensorNN::AvgPool2D(pd);
    }
    write_tensor("O", pd->O);
    return 0;
}

static int run_bn() {
    // params: N C H W eps affine
    auto p = read_params();
    auto s = ints(p, 0, 4);
    float eps = (float)atof(p[4].c_str());
    bool affine = atoi(p[5].c_str()) != 0;
    Tensor *x = gpu_tensor({s[0], s[1], s[2], s[3]}, "I.bin");
    Tensor *mean = gpu_tensor({s[1]}, "mean.bin"), *var = gpu_tensor({s[1]}, "var.bin");
    Tensor *g = affine ? gpu_tensor({s[1]}, "g.bin") : nullptr, *b = affine ? gpu_tensor({s[1]}, "b.bin") : nullptr;
    Tensor *y = new Tensor(x->getShape(), x->device), *opa = new Tensor(x->getShape(), x->device);
    Tensor *bn_mean = Tensor::zeros({s[1]}, x->device), *bn_var = Tensor::zeros({s[1]}, x->device);
    tensorNN::BatchNormForward(x, y, opa, mean, var, g, b, bn_mean, bn_var, /*trmode=*/false, eps, 0.99f);
    write_tensor("O", y);
    if (affine) write_tensor("opa", opa);
    write_tensor("bn_var", bn_var);
    return 0;
}

// UpSampling2D x2 -> Pad(0,1,1,0) -> Concat(skip) -> Add(itself) -> ReLU -> reshape -> Dense -> Softmax
static int run_chain() {
    // params: N C H W ndim
    auto p = read_params();
    auto s = ints(p, 0, 5);
    const int N = s[0], C = s[1], H = s[2], W = s[3], ndim = s[4];
    Tensor *x = gpu_tensor({N, C, H, W}, "I.bin");
    Tensor *skip = gpu_tensor({N, C, 2 * H + 1, 2 * W + 1}, "skip.bin");
    Tensor *up = new Tensor({N, C, 2 * H, 2 * W}, x->device);
    Tensor::scale(x, up, {2 * H, 2 * W});
    Tensor *padded = Tensor::zeros({N, C, 2 * H + 1, 2 * W + 1}, x->device);
    Tensor::pad(up, padded, {0, 1, 1, 0});
    Tensor *cat = Tensor::concat({skip, padded}, 1);
    Tensor *sum = new Tensor(cat->getShape(), x->device);
    Tensor::add(1.0f, cat, 1.0f, cat, sum, 0);
    Tensor *nadd = new Tensor(cat->getShape(), x->device);  // the n-ary Add layer: fill_(0) then inc per parent
    nadd->fill_(0.0f);
    Tensor::inc(cat, nadd);
    Tensor::inc(sum, nadd);
    Tensor *act = new Tensor(cat->getShape(), x->device);
    tensorNN::ReLu(nadd, act);
    write_tensor("cat", cat);
    const int feat = 2 * C * (2 * H + 1) * (2 * W + 1);
    act->reshape_({N, feat});
    Tensor *Wd = gpu_tensor({feat, ndim}, "W.bin"), *bd = gpu_tensor({ndim}, "b.bin");
    Tensor *dense = new Tensor({N, ndim}, x->device);
    Tensor::mult2D(act, 0, Wd, 0, dense, 0);
    Tensor::sum2D_rowwise(dense, bd, dense);
    Tensor *prob = new Tensor({N, ndim}, x->device), *sig = new Tensor({N, ndim}, x->device);
    tensorNN::FullSoftmax(dense, prob, 1);
    tensorNN::Sigmoid(dense, sig);
    write_tensor("act", act);
    write_tensor("dense", dense);
    write_tensor("prob", prob);
    write_tensor("sig", sig);
    return 0;
}

template <class F>
static bool throws(const char *what, const char *needle, F f) {
    try {
        f();
    } catch (const std::runtime_error &e) {
        if (std::string(e.what()).find(needle) != std::string::npos) return true;
        std::printf("FAIL %s: wrong message '%s'\n", what, e.what());
        return false;
    }
    std::printf("FAIL %s: no exception\n", what);
    return false;
}

static int run_errors() {
    bool ok = true;
    ok &= throws("bad padding name", "RuntimeError: ConvolDescriptor::ConvolDescriptor",
                 [] { ConvolDescriptor(4, {3, 3}, {1, 1}, "bogus", {}, 1, {1, 1}, true); });
    ok &= throws("grouped conv", "RuntimeError: ConvolDescriptor::ConvolDescriptor",
                 [] { ConvolDescriptor(4, {3, 3}, {1, 1}, "same", {}, 2, {1, 1}, true); });
    ok &= throws("bad device", "[HIP ERROR]", [] { gpu_init(99); });
    Tensor *x = Tensor::ones({1, 3, 4, 4}, DEV_GPU);
    ok &= throws("non 4D build", "RuntimeError: ConvolDescriptor::build", [&] {
        Tensor t({3, 4}, DEV_GPU);
        ConvolDescriptor cd(4, {3, 3}, {1, 1}, "same", {}, 1, {1, 1}, true);
        cd.build(&t);
    });
    ok &= throws("empty output", "RuntimeError: ConvolDescriptor::build", [&] {
        ConvolDescriptor cd(4, {5, 5}, {1, 1}, "valid", {}, 1, {1, 1}, true);
        cd.build(x);
    });
    ok &= throws("dilation", "RuntimeError: Tensor::Conv2D", [&] {
        ConvolDescriptor cd(4, {3, 3}, {1, 1}, "same", {}, 1, {2, 2}, true);
        cd.build(x);
        tensorNN::Conv2D(&cd);
    });
    ok &= throws("training-mode bn", "RuntimeError: gpu_batchnorm_forward", [&] {
        Tensor y(x->getShape(), DEV_GPU), m({3}, DEV_GPU), v({3}, DEV_GPU);
        tensorNN::BatchNormForward(x, &y, nullptr, &m, &v, nullptr, nullptr, &m, &v, true, 1e-5f, 0.9f);
    });
    ok &= throws("concat shape", "RuntimeError: Tensor::concat", [&] {
        Tensor y({1, 3, 5, 4}, DEV_GPU);
        Tensor::concat({x, &y}, 1);
    });
    ok &= throws("cpu tensor on the gpu backend", "RuntimeError: Tensor::ReLu", [&] {
        Tensor a({4}, DEV_CPU), b({4}, DEV_CPU);
        tensorNN::ReLu(&a, &b);
    });
    // a batch resize re-creates the storage (pointer churn the backend must tolerate)
    ConvolDescriptor cd(4, {3, 3}, {1, 1}, "same", {}, 1, {1, 1}, false);
    cd.build(x);
    cd.K->fill_(1.0f);
    tensorNN::Conv2D(&cd);
    x->resize(3);
    x->fill_(1.0f);
    cd.resize(3);
    tensorNN::Conv2D(&cd);
    cd.O->toCPU();
    ok &= cd.O->shape[0] == 3 && cd.O->ptr[5] == 27.0f && cd.O->ptr[2 * 4 * 16 + 0] == 12.0f;
    std::printf(ok ? "errors OK\n" : "errors FAILED\n");
    return ok ? 0 : 1;
}

int main(int argc, char **argv) {
    if (argc < 3) {
        std::fprintf(stderr, "usage: host_driver <case> <dir>\n");
        return 2;
    }
    std::string which = argv[1];
    g_dir = argv[2];
    try {
        if (which == "conv2d") return run_conv2d();
        if (which == "mpool") return run_pool(true);
        if (which == "avgpool") return run_pool(false);
        if (which == "bn") return run_bn();
        if (which == "chain") return run_chain();
        if (which == "errors") return run_errors();
    } catch (const std::exception &e) {
        std::fprintf(stderr, "host_driver: %s\n", e.what());
        return 3;
    }
    std::fprintf(stderr, "unknown case %s\n", which.c_str());
    return 2;
}
