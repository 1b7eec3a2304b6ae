// Model-level test driver of the C++ host layer: builds one of the benchmark graphs with the
// eddl:: API (the same constructions, in the same order, as eddl_amd/models.py), loads its
// parameters from a "bin" file, runs predict on an input read from a raw float file and writes
// the outputs to another.  The Python test compares the result with the Python graph runner on
// the same parameters, bit for bit.
//
// usage: net_driver <block|vgg16|resnet50|unet> <params.bin|-> <input.raw> <output.raw> <batch> <size> [model arguments]
//        net_driver errors
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <chrono>
#include <fstream>
#include <iostream>

#include "../../include/eddlhip.h"
#include "eddl_hip_net.h"
#include "eddl_hip_onnx.h"
#include "eddl_hip_synth.h"

using namespace eddl_hip;
using namespace eddl_hip::eddl;

static layer bn(layer l) { return BatchNormalization(l, true, 0.99f, 1e-5f); }

static model block(int channels, int size, int filters) {
    layer x = Input({channels, size, size});
    layer l = Conv2D(x, filters, {3, 3}, {1, 1}, "same", false);
    l = MaxPool2D(ReLu(bn(l)), {2, 2}, {2, 2}, "none");
    return Model({x}, {l});
}

static model vgg16(int size, int num_classes, const vector<int> &widths, int dense) {
    layer x = Input({3, size, size});
    layer l = x;
    const int reps[5] = {2, 2, 3, 3, 3};
    for (int s = 0; s < 5; s++) {
        for (int r = 0; r < reps[s]; r++) l = ReLu(Conv2D(l, widths[s], {3, 3}, {1, 1}, "same", true));
        l = MaxPool2D(l, {2, 2}, {2, 2}, "none");
    }
    l = Flatten(l);
    l = ReLu(Dense(l, dense));
    l = ReLu(Dense(l, dense));
    l = Softmax(Dense(l, num_classes));
    return Model({x}, {l});
}

static model resnet50(int size, int num_classes, int base) {
    const int stages[4] = {3, 4, 6, 3};
    layer x = Input({3, size, size});
    layer l = ReLu(bn(new LConv(x, base, {7, 7}, {2, 2}, "custom", {3, 3, 3, 3}, 1, {1, 1}, false, "")));
    l = new LMaxPool(l, vector<int>{3, 3}, vector<int>{2, 2}, vector<int>{1, 1, 1, 1}, "");
    int width = base;
    for (int si = 0; si < 4; si++) {
        for (int bi = 0; bi < stages[si]; bi++) {
            const int stride = (bi == 0 && si > 0) ? 2 : 1;
            const int out_ch = width * 4;
            layer sc = l;
            if (bi == 0) sc = bn(Conv2D(l, out_ch, {1, 1}, {stride, stride}, "valid", false));
            layer m = ReLu(bn(Conv2D(l, width, {1, 1}, {1, 1}, "valid", false)));
            if (stride == 1) m = Conv2D(m, width, {3, 3}, {1, 1}, "same", false);
            else m = new LConv(m, width, {3, 3}, {2, 2}, "custom", {1, 1, 1, 1}, 1, {1, 1}, false, "");
            m = ReLu(bn(m));
            m = bn(Conv2D(m, out_ch, {1, 1}, {1, 1}, "valid", false));
            l = ReLu(Add(m, sc));
        }
        width *= 2;
    }
    l = Dense(Flatten(GlobalAveragePool2D(l)), num_classes);
    return Model({x}, {l});
}

static layer twice(layer l, int w) {
    for (int i = 0; i < 2; i++) l = ReLu(bn(Conv2D(l, w, {3, 3}, {1, 1}, "same", true)));
    return l;
}

static model unet(int size, const vector<int> &widths, int bottleneck) {
    layer x = Input({1, size, size});
    layer l = x;
    vector<layer> skips;
    for (int w : widths) {
        l = twice(l, w);
        skips.push_back(l);
        l = MaxPool2D(l, {2, 2}, {2, 2}, "none");
    }
    l = twice(l, bottleneck);
    for (size_t i = widths.size(); i-- > 0;) {
        l = UpSampling2D(l, {2, 2});
        l = Conv2D(Pad(l, {0, 1, 1, 0}), widths[i], {2, 2}, {1, 1}, "valid", true);
        l = Concat({skips[i], l});
        l = twice(l, widths[i]);
    }
    l = Sigmoid(Conv2D(l, 1, {1, 1}, {1, 1}, "valid", true));
    return Model({x}, {l});
}

template <class F>
static bool throws(F f, const char *what) {
    try {
        f();
    } catch (const std::exception &e) {
        printf("ok %s: %s\n", what, e.what());
        return true;
    }
    printf("FAILED %s: no exception\n", what);
    return false;
}

static int errors() {
    bool ok = true;
    ok &= throws([] { Conv2D(Input({3, 224, 224}), 64, {7, 7}, {2, 2}, "same"); }, "asymmetric 7x7 s2 same");
    try {
        Conv2D(Input({3, 8, 8}), 4, {2, 2}, {1, 1}, "same");
        ok = false;
    } catch (const AsymmetricPaddingException &e) {
        vector<int> p = e.get_asymmetric_pads();
        printf("ok asymmetric pads %d %d %d %d\n", p[0], p[1], p[2], p[3]);
        ok &= p == vector<int>({0, 1, 0, 1});
    }
    try {  // pools refuse asymmetric paddings as well: "same" 2x2 stride 2 on an odd plane pads (0,1)
        MaxPool2D(Input({3, 5, 5}), {2, 2}, {2, 2}, "same");
        ok = false;
        printf("FAILED asymmetric pool pads: no exception\n");
    } catch (const AsymmetricPaddingException &e) {
        vector<int> p = e.get_asymmetric_pads();
        printf("ok asymmetric pool pads %d %d %d %d\n", p[0], p[1], p[2], p[3]);
        ok &= p == vector<int>({0, 1, 0, 1});
    }
    ok &= throws([] { AveragePool2D(Input({3, 5, 5}), {2, 2}, {2, 2}, "same"); }, "asymmetric average pool");
    ok &= throws([] { Dense(Input({4}), 3)->forward(); }, "forward before build");
    ok &= throws([] { Reshape(Input({4, 4}), {-1, -1}); }, "ambiguous reshape");
    ok &= throws([] { Reshape(Input({4, 4}), {5}); }, "incompatible reshape");
    ok &= throws([] { Concat({Input({4, 4, 4})}); }, "concat of one layer");
    ok &= throws([] { Concat({Input({4, 4, 4}), Input({4, 5, 4})}); }, "concat of different planes");
    ok &= throws([] { Add(Input({4, 4, 4}), Input({4, 5, 4})); }, "add of different shapes");
    ok &= throws([] { Softmax(Input({4}), 0); }, "softmax over the batch");
    ok &= throws([] { Activation(Input({4}), "elu"); }, "activation outside the path");
    ok &= throws([] {
        model m = block(3, 8, 4);
        build(m, CS_HIP({1, 1}));
    }, "two GPUs");
    ok &= throws([] {
        model m = block(3, 8, 4);
        build(m, CS_HIP({1}));
        load(m, "/nonexistent/file.bin");
    }, "missing parameter file");
    ok &= throws([] {
        model m = block(3, 8, 4);
        build(m, CS_HIP({1}));
        Tensor a({2, 3, 8, 8}), b({2, 3, 8, 8});
        predict(m, {&a, &b});
    }, "two inputs for one input layer");
    ok &= throws([] {  // the fused plan calls the library past tensorNN::Conv2D: it has to refuse dilations itself
        layer x = Input({3, 12, 12});
        model m = Model({x}, {ReLu(Conv2D(x, 4, {3, 3}, {1, 1}, "same", true, 1, {2, 2}))});
        build(m, CS_HIP({1}));
        fuse(m);
        Tensor a({2, 3, 12, 12});
        predict(m, {&a});
    }, "dilated convolution in a fused plan");
    ok &= throws([] {  // a batch norm absorbed into a convolution step must not run as inference in training mode
        model m = block(3, 8, 4);
        build(m, CS_HIP({1}));
        fuse(m);
        set_mode(m, TRMODE);
        Tensor a({2, 3, 8, 8});
        forward(m, {&a});
    }, "training-mode batch norm in a fused plan");
    return ok ? 0 : 1;
}

// onnx <file.onnx> <input.raw> <output.raw> <batch> <fused 0|1> [<re-export.onnx>]: imports the file, runs one
// batch, writes the output; with a last argument also writes the built net back out as ONNX.
static int onnx(int argc, char **argv) {
    if (argc < 7) {
        fprintf(stderr, "usage: net_driver onnx <file.onnx> <input.raw> <output.raw> <batch> <fused> [<re-export.onnx>]\n");
        return 2;
    }
    try {
        model m = eddl_hip::import_net_from_onnx_file(argv[2]);
        printf("layers:");
        for (Layer *l : m->layers) printf(" %s", l->kind().c_str());
        printf("\nnames:");
        for (Layer *l : m->layers) printf(" %s", l->name.c_str());
        printf("\n");
        build(m, CS_HIP({1}), false);  // keep the imported parameters
        if (atoi(argv[6])) {
            fuse(m);
            printf("plan: %zu steps\n", m->plan.size());
        }
        vector<int> ishape = m->lin[0]->output->getShape();
        ishape[0] = atoi(argv[5]);
        Tensor x(ishape, DEV_CPU);
        std::ifstream ifs(argv[3], std::ios::binary);
        ifs.read(reinterpret_cast<char *>(x.ptr), x.size * sizeof(float));
        if (!ifs.good()) {
            fprintf(stderr, "short input file\n");
            return 2;
        }
        vtensor out = predict(m, {&x});
        std::ofstream ofs(argv[4], std::ios::binary);
        for (Tensor *t : out) {
            ofs.write(reinterpret_cast<const char *>(t->ptr), t->size * sizeof(float));
            delete t;
        }
        if (argc > 7) eddl_hip::save_net_to_onnx_file(m, argv[7]);
        bool threw = false;
        try {
            eddl_hip::import_net_from_onnx_file(string(argv[2]) + ".absent");
        } catch (const std::runtime_error &) {
            threw = true;
        }
        printf("%s missing ONNX file\n", threw ? "ok " : "FAILED");
        delete m;
    } catch (const std::exception &e) {
        fprintf(stderr, "exception: %s\n", e.what());
        return 1;
    }
    return 0;
}

// onnxinfo <file.onnx> [<re-export.onnx>]: imports the file on the host (no GPU is touched) and prints one line
// per layer: kind, name, output shape, and per parameter its size and the sum of its values; with a second
// argument the imported net is written back out as ONNX.
static int onnxinfo(int argc, char **argv) {
    if (argc < 3) {
        fprintf(stderr, "usage: net_driver onnxinfo <file.onnx> [<re-export.onnx>]\n");
        return 2;
    }
    try {
        model m = eddl_hip::import_net_from_onnx_file(argv[2]);
        for (Layer *l : m->layers) {
            printf("layer %s %s", l->kind().c_str(), l->name.c_str());
            for (int d : l->output->shape) printf(" %d", d);
            for (Tensor *t : l->params) {
                double sum = 0.0;
                for (unsigned long i = 0; i < t->size; i++) sum += t->ptr[i];
                printf(" | %lu %.9g", t->size, sum);
            }
            printf("\n");
        }
        if (argc > 3) eddl_hip::save_net_to_onnx_file(m, argv[3]);
        delete m;
    } catch (const std::exception &e) {
        fprintf(stderr, "exception: %s\n", e.what());
        return 1;
    }
    return 0;
}

// net_driver loadbin <model> <params.bin> <size> [model arguments]: the graph is made but not built (its parameters are
// host tensors), the file is read into it, and every parameter's size and sum are printed - the bin reader alone, no device.
static int loadbin(int argc, char **argv) {
    if (argc < 5) {
        fprintf(stderr, "usage: net_driver loadbin <model> <params.bin> <size> [model arguments]\n");
        return 2;
    }
    const string which = argv[2];
    const int size = atoi(argv[4]);
    vector<int> extra;
    for (int i = 5; i < argc; i++) extra.push_back(atoi(argv[i]));
    try {
        model m = nullptr;
        if (which == "block") m = block(extra.at(0), size, extra.at(1));
        else if (which == "vgg16") m = vgg16(size, extra.at(0), {extra.at(1), extra.at(2), extra.at(3), extra.at(4), extra.at(5)}, extra.at(6));
        else if (which == "resnet50") m = resnet50(size, extra.at(0), extra.at(1));
        else if (which == "unet") m = unet(size, vector<int>(extra.begin(), extra.end() - 1), extra.back());
        else {
            fprintf(stderr, "unknown model %s\n", which.c_str());
            return 2;
        }
        load(m, argv[3]);
        for (Layer *l : m->layers)
            for (Tensor *t : l->params) {
                double sum = 0.0;
                for (unsigned long i = 0; i < t->size; i++) sum += t->ptr[i];
                printf("param %s %lu %.9g\n", l->name.c_str(), t->size, sum);
            }
        delete m;
    } catch (const std::exception &e) {
        fprintf(stderr, "exception: %s\n", e.what());
        return 1;
    }
    return 0;
}

int main(int argc, char **argv) {
    if (argc >= 2 && !strcmp(argv[1], "errors")) return errors();
    if (argc >= 2 && !strcmp(argv[1], "loadbin")) return loadbin(argc, argv);
    if (argc >= 2 && !strcmp(argv[1], "onnxinfo")) return onnxinfo(argc, argv);
    if (argc >= 2 && !strcmp(argv[1], "onnx")) return onnx(argc, argv);
    if (argc < 7) {
        fprintf(stderr, "usage: net_driver <model> <params.bin|-> <input.raw> <output.raw> <batch> <size> [model arguments]\n");
        return 2;
    }
    // <model> may carry flags in front: "fused:vgg16", "time:vgg16", "fused+time:vgg16"
    string which = argv[1];
    bool fused = false, timed = false;
    const size_t colon = which.find(':');
    if (colon != string::npos) {
        const string flags = which.substr(0, colon);
        fused = flags.find("fused") != string::npos;
        timed = flags.find("time") != string::npos;
        which = which.substr(colon + 1);
    }
    const string params = argv[2], in_path = argv[3], out_path = argv[4];
    const int batch = atoi(argv[5]), size = atoi(argv[6]);
    // (the binding's gpu_init switches the library's plan search on unless EDDLHIP_NO_TUNE is set, and starts it from the
    // plans in EDDLHIP_PLANS=<file>; EDDLHIP_PLANS_SAVE=<file> makes this driver write the table it ends up with)
    vector<int> extra;
    for (int i = 7; i < argc; i++) extra.push_back(atoi(argv[i]));
    try {
        model m = nullptr;
        if (which == "block") m = block(extra.at(0), size, extra.at(1));
        else if (which == "vgg16") m = vgg16(size, extra.at(0), {extra.at(1), extra.at(2), extra.at(3), extra.at(4), extra.at(5)}, extra.at(6));
        else if (which == "resnet50") m = resnet50(size, extra.at(0), extra.at(1));
        else if (which == "unet") m = unet(size, vector<int>(extra.begin(), extra.end() - 1), extra.back());
        else {
            fprintf(stderr, "unknown model %s\n", which.c_str());
            return 2;
        }
        // parameters "synth:<seed>": drawn on the host by the generator the Python host shares, then moved to the device;
        // "-": drawn on the device by build(); anything else: a bin file loaded after build
        const bool synth_params = params.compare(0, 6, "synth:") == 0;
        if (synth_params) eddl_hip::synth_he_normal(m, (uint32_t)strtoul(params.c_str() + 6, nullptr, 10));
        build(m, CS_HIP({1}), !synth_params);
        if (getenv("EDDLHIP_PLANS") != nullptr && getenv("EDDLHIP_PLANS")[0] != 0) printf("plans: %d geometries loaded\n", eddlhip_conv2d_tuned_plans(0));
        if (fused) {
            fuse(m);
            int away = 0;
            for (Layer *l : m->layers) away += m->is_fused_away(l) ? 1 : 0;
            printf("plan: %zu steps, %d layers computed inside another layer's step\n", m->plan.size(), away);
        }
        if (params != "-" && !synth_params) load(m, params);  // after fuse(): the kept filter copies must follow the new values
        printf("layers:");
        for (Layer *l : m->layers) printf(" %s", l->kind().c_str());
        printf("\n");
        vector<int> ishape = m->lin[0]->output->getShape();
        ishape[0] = batch;
        Tensor x(ishape, DEV_CPU);
        if (in_path.compare(0, 6, "synth:") == 0) {  // synth:<seed>:<uniform|normal>: no input file either
            const size_t colon2 = in_path.find(':', 6);
            eddl_synth *gen = eddl_synth_new((uint32_t)strtoul(in_path.substr(6, colon2 - 6).c_str(), nullptr, 10));
            if (in_path.substr(colon2 + 1) == "uniform") eddl_synth_uniform(gen, x.ptr, x.size, 0.0f, 1.0f);
            else eddl_synth_normal(gen, x.ptr, x.size, 0.0f, 1.0f);
            eddl_synth_free(gen);
        } else {
            std::ifstream ifs(in_path, std::ios::binary);
            ifs.read(reinterpret_cast<char *>(x.ptr), x.size * sizeof(float));
            if (!ifs.good()) {
                fprintf(stderr, "short input file\n");
                return 2;
            }
        }
        // two forwards at two batch sizes first: every tensor is re-created on the way (resize)
        if (batch > 1) {
            vector<int> one = ishape;
            one[0] = 1;
            Tensor x1(one, DEV_CPU);
            memcpy(x1.ptr, x.ptr, x1.size * sizeof(float));
            for (Tensor *t : predict(m, {&x1})) delete t;
        }
        vtensor out = predict(m, {&x});
        std::ofstream ofs(out_path, std::ios::binary);
        for (Tensor *t : out) {
            printf("output");
            for (int d : t->shape) printf(" %d", d);
            printf("\n");
            ofs.write(reinterpret_cast<const char *>(t->ptr), t->size * sizeof(float));
            delete t;
        }
        ofs.close();
        show_profile();
        if (timed) {  // forwards with the input already on the device
            // warm-up: at least five forwards and 0.2 s, so that the device's clocks have settled
            const auto w0 = std::chrono::steady_clock::now();
            for (int i = 0; i < 5 || std::chrono::duration<double>(std::chrono::steady_clock::now() - w0).count() < 0.2; i++) m->forward();
            const auto t0 = std::chrono::steady_clock::now();
            const int reps = 20;
            for (int i = 0; i < reps; i++) m->forward();
            const double ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count() / reps;
            size_t ws = 0;
            eddlhip_workspace_bytes(0, &ws);
            printf("ms_per_forward %.4f images_per_s %.1f workspace_bytes %zu tuned_geometries %d\n", ms, batch * 1000.0 / ms, ws, eddlhip_conv2d_tuned_plans(0));
        }
        if (fused) {  // a layer inside a chain has no output to hand out
            for (Layer *l : m->layers)
                if (m->is_fused_away(l)) {
                    bool threw = false;
                    try {
                        delete getOutput(l);
                    } catch (const std::runtime_error &) {
                        threw = true;
                    }
                    printf("%s getOutput of a fused-away layer\n", threw ? "ok " : "FAILED");
                    break;
                }
        }
        {  // parameters out and back in: a doubled bias-free copy changes the result, the original restores it
            vector<vtensor> ps = get_parameters(m);
            size_t count = 0;
            for (vtensor &v : ps) count += v.size();
            set_parameters(m, ps);
            vtensor again = predict(m, {&x});
            bool same = true;
            {
                std::ifstream chk(out_path, std::ios::binary);
                for (Tensor *t : again) {
                    vector<float> ref(t->size);
                    chk.read(reinterpret_cast<char *>(ref.data()), t->size * sizeof(float));
                    same = same && memcmp(ref.data(), t->ptr, t->size * sizeof(float)) == 0;
                    delete t;
                }
            }
            printf("%s get_parameters / set_parameters round trip (%zu tensors)\n", same ? "ok " : "FAILED", count);
            bool threw = false;
            try {
                vector<vtensor> fewer(ps.begin(), ps.end() - 1);
                set_parameters(m, fewer);
            } catch (const std::runtime_error &) {
                threw = true;
            }
            printf("%s set_parameters with a missing layer\n", threw ? "ok " : "FAILED");
            printf("%s getLayer / getOut\n", getLayer(m, m->layers.back()->name) == m->layers.back() && getOut(m) == m->lout ? "ok " : "FAILED");
            for (vtensor &v : ps)
                for (Tensor *t : v) delete t;
        }
        if (params == "-") save(m, out_path + ".params");  // round trip of freshly initialised parameters
        delete m;
        const char *plans_out = getenv("EDDLHIP_PLANS_SAVE");
        if (plans_out != nullptr && plans_out[0] != 0 && eddlhip_conv2d_tuned_save(0, plans_out) != 0) {
            fprintf(stderr, "plans: %s\n", eddlhip_last_error());
            return 2;
        }
    } catch (const std::exception &e) {
        fprintf(stderr, "exception: %s\n", e.what());
        return 1;
    }
    return 0;
}
