// ONNX import / export of the forward path (see eddl_hip_onnx.h for what it mirrors).
//
// Wire format: a message is a sequence of fields, each a varint key (field number << 3 | wire type)
// followed by a varint (type 0), 8 bytes (1), a varint length and that many bytes (2) or 4 bytes (5).
// Field numbers are the ones of onnx.proto (the file the reference vendors under
// src/serialization/onnx/onnx_third_party/).
#include "eddl_hip_onnx.h"

#include <cstdint>
#include <cstring>
#include <deque>
#include <fstream>
#include <iostream>
#include <map>
#include <set>
#include <sstream>

namespace eddl_hip {
namespace {

// ---------------------------------------------------------------- reading
struct Span {
    const uint8_t *p = nullptr;
    size_t n = 0;
};

struct ParseError : std::runtime_error {
    using std::runtime_error::runtime_error;
};

struct Field {
    int number = 0, wire = 0;
    uint64_t value = 0;  // wire types 0, 1, 5
    Span bytes;          // wire type 2
};

class Reader {
  public:
    explicit Reader(Span s) : cur(s.p), end(s.p + s.n) {}
    bool next(Field &f) {
        if (cur >= end) return false;
        const uint64_t key = varint();
        f.number = (int)(key >> 3);
        f.wire = (int)(key & 7);
        f.value = 0;
        f.bytes = Span();
        switch (f.wire) {
            case 0: f.value = varint(); break;
            case 1: f.value = fixed(8); break;
            case 5: f.value = fixed(4); break;
            case 2: {
                const uint64_t len = varint();
                if (len > (uint64_t)(end - cur)) throw ParseError("truncated length-delimited field");
                f.bytes.p = cur;
                f.bytes.n = (size_t)len;
                cur += len;
                break;
            }
            default: throw ParseError("unsupported wire type");
        }
        return true;
    }
    uint64_t varint() {
        uint64_t v = 0;
        for (int shift = 0; shift < 64; shift += 7) {
            if (cur >= end) throw ParseError("truncated varint");
            const uint8_t b = *cur++;
            v |= (uint64_t)(b & 0x7F) << shift;
            if (!(b & 0x80)) return v;
        }
        throw ParseError("varint longer than 64 bits");
    }

  private:
    uint64_t fixed(int bytes) {
        if (end - cur < bytes) throw ParseError("truncated fixed-width field");
        uint64_t v = 0;
        memcpy(&v, cur, bytes);  // little endian on both sides
        cur += bytes;
        return v;
    }
    const uint8_t *cur, *end;
};

string text(const Span &s) { return string(reinterpret_cast<const char *>(s.p), s.n); }

void packed_ints(const Field &f, vector<int64_t> &out) {
    if (f.wire != 2) {
        out.push_back((int64_t)f.value);
        return;
    }
    const uint8_t *q = f.bytes.p, *stop = f.bytes.p + f.bytes.n;  // a packed run: varints back to back
    while (q < stop) {
        uint64_t v = 0;
        int shift = 0;
        for (;;) {
            if (q >= stop) throw ParseError("truncated packed varint");
            const uint8_t b = *q++;
            v |= (uint64_t)(b & 0x7F) << shift;
            if (!(b & 0x80)) break;
            shift += 7;
            if (shift > 63) throw ParseError("varint longer than 64 bits");
        }
        out.push_back((int64_t)v);
    }
}

template <typename T>
void packed_fixed(const Field &f, vector<T> &out) {
    if (f.wire == 2) {
        const size_t count = f.bytes.n / sizeof(T);
        const size_t at = out.size();
        out.resize(at + count);
        memcpy(out.data() + at, f.bytes.p, count * sizeof(T));
    } else {
        T v;
        memcpy(&v, &f.value, sizeof(T));
        out.push_back(v);
    }
}

enum DataType { FLOAT = 1, UINT8 = 2, INT8 = 3, UINT16 = 4, INT16 = 5, INT32 = 6, INT64 = 7, BOOL = 9, DOUBLE = 11 };

// TensorProto: dims 1, data_type 2, float_data 4, int32_data 5, int64_data 7, name 8, raw_data 9, double_data 10.
// Every type becomes floats, as parseTensorValues does (src/serialization/onnx/net/utils_onnx.cpp:24-120).
struct TensorP {
    string name;
    vector<int> dims;
    int data_type = 0;
    vector<float> values;

    TensorP() {}
    explicit TensorP(Span s) {
        vector<int64_t> d, i32, i64;
        vector<float> f32;
        vector<double> f64;
        Span raw;
        bool has_raw = false;
        Reader r(s);
        Field f;
        while (r.next(f)) {
            if (f.number == 1) packed_ints(f, d);
            else if (f.number == 2) data_type = (int)f.value;
            else if (f.number == 4) packed_fixed(f, f32);
            else if (f.number == 5) packed_ints(f, i32);
            else if (f.number == 7) packed_ints(f, i64);
            else if (f.number == 8) name = text(f.bytes);
            else if (f.number == 9) { raw = f.bytes; has_raw = true; }
            else if (f.number == 10) packed_fixed(f, f64);
        }
        for (int64_t v : d) dims.push_back((int)v);
        if (has_raw) {
            auto take = [&](auto sample) {
                typedef decltype(sample) T;
                const size_t count = raw.n / sizeof(T);
                values.resize(count);
                for (size_t i = 0; i < count; i++) {
                    T v;
                    memcpy(&v, raw.p + i * sizeof(T), sizeof(T));
                    values[i] = (float)v;
                }
            };
            switch (data_type) {
                case FLOAT: take(float()); break;
                case DOUBLE: take(double()); break;
                case INT64: take(int64_t()); break;
                case INT32: take(int32_t()); break;
                case INT16: take(int16_t()); break;
                case UINT16: take(uint16_t()); break;
                case INT8: take(int8_t()); break;
                case UINT8: case BOOL: take(uint8_t()); break;
                default: break;
            }
        } else if (data_type == FLOAT) {
            values = f32;
        } else if (data_type == INT64) {
            for (int64_t v : i64) values.push_back((float)v);
        } else if (data_type == DOUBLE) {
            for (double v : f64) values.push_back((float)v);
        } else {
            for (int64_t v : i32) values.push_back((float)v);
        }
    }
};

// AttributeProto: name 1, f 2, i 3, s 4, t 5, floats 7, ints 8
struct AttrP {
    string name, s;
    float f = 0.0f;
    int64_t i = 0;
    bool has_t = false;
    TensorP t;
    vector<float> floats;
    vector<int64_t> ints;
    explicit AttrP(Span sp) {
        Reader r(sp);
        Field fd;
        while (r.next(fd)) {
            if (fd.number == 1) name = text(fd.bytes);
            else if (fd.number == 2) { uint32_t u = (uint32_t)fd.value; memcpy(&f, &u, 4); }
            else if (fd.number == 3) i = (int64_t)fd.value;
            else if (fd.number == 4) s = text(fd.bytes);
            else if (fd.number == 5) { t = TensorP(fd.bytes); has_t = true; }
            else if (fd.number == 7) packed_fixed(fd, floats);
            else if (fd.number == 8) packed_ints(fd, ints);
        }
    }
    vector<int> int_list() const { return vector<int>(ints.begin(), ints.end()); }
};

// NodeProto: input 1, output 2, name 3, op_type 4, attribute 5
struct NodeP {
    vector<string> input, output, positional;
    string name, op_type;
    vector<AttrP> attribute;
    explicit NodeP(Span sp) {
        Reader r(sp);
        Field f;
        while (r.next(f)) {
            if (f.number == 1) input.push_back(text(f.bytes));
            else if (f.number == 2) output.push_back(text(f.bytes));
            else if (f.number == 3) name = text(f.bytes);
            else if (f.number == 4) op_type = text(f.bytes);
            else if (f.number == 5) attribute.emplace_back(f.bytes);
        }
    }
    const AttrP *attr(const string &n) const {
        for (const AttrP &a : attribute)
            if (a.name == n) return &a;
        return nullptr;
    }
};

// ValueInfoProto: name 1, type 2 { tensor_type 1 { elem_type 1, shape 2 { dim 1 { dim_value 1, dim_param 2 } } } }
struct ValueInfoP {
    string name;
    vector<int> dims;  // -1 for a symbolic dimension
    explicit ValueInfoP(Span sp) {
        Reader r(sp);
        Field f;
        while (r.next(f)) {
            if (f.number == 1) name = text(f.bytes);
            if (f.number != 2) continue;
            Reader r2(f.bytes);
            Field f2;
            while (r2.next(f2)) {
                if (f2.number != 1) continue;
                Reader r3(f2.bytes);
                Field f3;
                while (r3.next(f3)) {
                    if (f3.number != 2) continue;
                    Reader r4(f3.bytes);
                    Field f4;
                    while (r4.next(f4)) {
                        if (f4.number != 1) continue;
                        int dim = -1;
                        Reader r5(f4.bytes);
                        Field f5;
                        while (r5.next(f5))
                            if (f5.number == 1) dim = (int)(int64_t)f5.value;
                        dims.push_back(dim);
                    }
                }
            }
        }
    }
};

// GraphProto: node 1, name 2, initializer 5, input 11, output 12;  ModelProto: graph 7
struct GraphP {
    vector<NodeP> node;
    vector<TensorP> initializer;
    vector<ValueInfoP> input, output;
    explicit GraphP(Span model) {
        Reader rm(model);
        Field fm;
        bool found = false;
        while (rm.next(fm)) {
            if (fm.number != 7 || fm.wire != 2) continue;
            found = true;
            Reader r(fm.bytes);
            Field f;
            while (r.next(f)) {
                if (f.wire != 2) continue;
                if (f.number == 1) node.emplace_back(f.bytes);
                else if (f.number == 5) initializer.emplace_back(f.bytes);
                else if (f.number == 11) input.emplace_back(f.bytes);
                else if (f.number == 12) output.emplace_back(f.bytes);
            }
        }
        if (!found) throw ParseError("the file holds no graph");
    }
};

void info(const string &s) { std::cerr << "[ONNX::INFO] " << s << std::endl; }

// ---------------------------------------------------------------- import
class Importer {
  public:
    Importer(GraphP &g, const vector<int> &input_shape) : graph(g) {
        for (TensorP &t : g.initializer) {
            values[t.name] = t.values;
            dims[t.name] = t.dims;
        }
        for (NodeP &n : g.node)  // constant nodes are always available (initialize_constant_nodes)
            if (n.op_type == "Constant" && !n.output.empty()) {
                const AttrP *a = n.attr("value");
                if (a && a->has_t) {
                    values[n.output[0]] = a->t.values;
                    dims[n.output[0]] = a->t.dims;
                }
            }
        for (NodeP &n : g.node)
            for (const string &i : n.input) users[i].push_back(&n);
        for (ValueInfoP &vi : g.input)  // get_inputs (import_helpers.cpp:246-278)
            if (!values.count(vi.name)) true_inputs.push_back(&vi);
        if (true_inputs.empty()) msg("the graph has no input", "ONNX::ImportNet");
        if (!input_shape.empty()) {
            if (true_inputs.size() > 1)
                msg("The imported model has more than 1 input layer and the shape provided to reshape the model can only be applied"
                    "if the model has only one input layer.",
                    "ONNX::ImportNet");
            inputs.push_back(eddl::Input(input_shape, true_inputs[0]->name));
        } else {
            for (ValueInfoP *vi : true_inputs) {
                vector<int> shape(vi->dims.begin() + (vi->dims.empty() ? 0 : 1), vi->dims.end());
                bool fixed = !shape.empty();
                for (int d : shape) fixed = fixed && d > 0;
                if (!fixed) msg("input " + vi->name + " has no fixed shape after the batch dimension; pass input_shape", "ONNX::ImportNet");
                inputs.push_back(eddl::Input(shape, vi->name));
            }
        }
    }

    // the queue walk of process_node_queue (import_helpers.cpp:529-598)
    Net *run() {
        std::deque<NodeP *> q;
        for (size_t i = 0; i < inputs.size(); i++) {
            layers[true_inputs[i]->name] = inputs[i];
            for (NodeP *u : users[true_inputs[i]->name]) q.push_back(u);
        }
        for (NodeP &n : graph.node) {  // nodes fed by initializers and constants only (queue_constant_nodes)
            if (n.op_type == "Constant" || n.input.empty()) continue;
            bool all = true;
            for (const string &i : n.input) all = all && (i.empty() || values.count(i));
            if (all) q.push_back(&n);
        }
        std::set<NodeP *> built;
        while (!q.empty()) {
            NodeP *n = q.front();
            q.pop_front();
            if (n->op_type == "Constant" || n->output.empty() || built.count(n) || layers.count(n->output[0])) continue;
            if (n->positional.empty()) {
                n->positional = n->input;  // Resize addresses its inputs by position
                vector<string> kept;       // empty names some exporters leave behind
                for (const string &i : n->input)
                    if (!i.empty()) kept.push_back(i);
                n->input = kept;
            }
            bool ready = true;
            for (const string &i : n->input) ready = ready && (values.count(i) || layers.count(i));
            if (!ready) continue;  // comes back when the missing input's producer is created
            built.insert(n);
            Layer *l = build(*n);
            for (const string &o : n->output) {
                if (l != nullptr) layers[o] = l;
                for (NodeP *u : users[o]) q.push_back(u);
            }
        }
        vector<Layer *> outs;
        for (ValueInfoP &vi : graph.output) {
            if (!layers.count(vi.name)) msg("graph output " + vi.name + " was not produced by any imported node", "ONNX::ImportNet");
            outs.push_back(layers[vi.name]);
        }
        return new Net(inputs, outs);
    }

  private:
    GraphP &graph;
    std::map<string, vector<float>> values;  // map_init_values
    std::map<string, vector<int>> dims;      // map_init_dims
    std::map<string, Layer *> layers;        // output_node_map
    std::map<string, vector<NodeP *>> users;  // input_node_map
    vector<ValueInfoP *> true_inputs;
    vector<Layer *> inputs;

    Layer *parent(const NodeP &n, size_t i = 0) {
        if (i >= n.input.size() || !layers.count(n.input[i]))
            msg("node " + n.name + " (" + n.op_type + "): input " + std::to_string(i) + " is not a layer", "ONNX::ImportNet");
        return layers[n.input[i]];
    }

    void fill(Tensor *t, const NodeP &n, size_t input_index) {
        if (input_index >= n.input.size() || !values.count(n.input[input_index]))
            msg("node " + n.name + ": parameter " + std::to_string(input_index) + " is not an initializer", "ONNX::ImportNet");
        const vector<float> &v = values[n.input[input_index]];
        if (v.size() != t->size)
            msg("node " + n.name + ": parameter " + n.input[input_index] + " holds " + std::to_string(v.size()) + " values, the layer needs " +
                    std::to_string(t->size),
                "Tensor::copy");
        memcpy(t->ptr, v.data(), v.size() * sizeof(float));
    }

    void need_4d(Layer *p, const NodeP &n) {
        if (p->output->ndim != 4) msg("node " + n.name + ": only the 2D form is on this backend's path", "ONNX::ImportNet");
    }

    Layer *build(NodeP &n) {
        const string &op = n.op_type;
        if (op == "Conv") return conv(n);
        if (op == "BatchNormalization") return batchnorm(n);
        if (op == "Relu") return new LActivation(parent(n), "relu", {}, n.name);
        if (op == "Sigmoid") return new LActivation(parent(n), "sigmoid", {}, n.name);
        if (op == "Softmax") return softmax(n);
        if (op == "MaxPool") return pool(n, true);
        if (op == "AveragePool") return pool(n, false);
        if (op == "GlobalAveragePool" || op == "GlobalMaxPool") {
            Layer *p = parent(n);
            need_4d(p, n);
            const vector<int> plane = {p->output->shape[2], p->output->shape[3]};
            if (op == "GlobalMaxPool") return new LMaxPool(p, plane, {1, 1}, string("none"), n.name);
            return new LAveragePool(p, plane, {1, 1}, string("none"), n.name);
        }
        if (op == "Gemm") return gemm(n);
        if (op == "MatMul") return dense(n, 0);
        if (op == "Add") return add(n);
        if (op == "Sum") {
            if (n.input.size() != 2 || values.count(n.input[1]))
                msg("Error: The second input summand of the Sum layer " + n.name + " is not valid", "ONNX::ImportNet");
            return new LSum(parent(n, 0), parent(n, 1), n.name);
        }
        if (op == "Concat") return concat(n);
        if (op == "Upsample") return upsample(n);
        if (op == "Resize") return resize(n);
        if (op == "Pad") return pad(n);
        if (op == "Flatten") return new LReshape(parent(n), {1, -1}, n.name);
        if (op == "Reshape") return reshape(n);
        if (op == "Identity") {
            if (layers.count(n.input[0])) return layers[n.input[0]];
            for (const string &o : n.output) {
                values[o] = values[n.input[0]];
                dims[o] = dims[n.input[0]];
            }
            return nullptr;
        }
        msg("The ONNX node type " + op + " (node " + n.name + ") is outside the forward path this backend implements", "ONNX::ImportNet");
        return nullptr;
    }

    // layers/conv/conv_onnx.cpp:6-213
    Layer *conv(const NodeP &n) {
        Layer *p = parent(n);
        need_4d(p, n);
        string auto_pad = "custom";
        vector<int> pads, strides, dilations;
        int groups = 1;
        for (const AttrP &a : n.attribute) {
            if (a.name == "auto_pad") {
                if (a.s == "NOTSET") auto_pad = "custom";
                else if (a.s == "VALID") auto_pad = "valid";
                else if (a.s == "SAME_UPPER" || a.s == "SAME_LOWER") auto_pad = "same";
            } else if (a.name == "dilations") dilations = a.int_list();
            else if (a.name == "group") groups = (int)a.i;
            else if (a.name == "pads") {
                pads = a.int_list();
                if (pads.size() == 4) std::swap(pads[1], pads[2]);  // [top, left, bottom, right] -> [top, bottom, left, right]
            } else if (a.name == "strides") strides = a.int_list();
        }
        if (n.input.size() < 2 || !values.count(n.input[1])) msg("node " + n.name + ": the filters are not an initializer", "ONNX::ImportNet");
        const vector<int> &wd = dims[n.input[1]];
        if (wd.size() != 4) msg("node " + n.name + ": the filters are not 4D", "ONNX::ImportNet");
        const vector<int> kernel = {wd[2], wd[3]};
        const bool use_bias = n.input.size() > 2;
        if (dilations.empty()) dilations = {1, 1};
        if (strides.empty()) strides = {1, 1};
        if (pads.empty() && auto_pad == "custom") pads = {0, 0, 0, 0};
        LConv *l = nullptr;
        try {
            l = new LConv(p, wd[0], kernel, strides, auto_pad, pads, groups, dilations, use_bias, n.name);
        } catch (const AsymmetricPaddingException &e) {
            info("Detected a padding asymmetry in layer " + n.name + ". Going to add an explicit Pad layer before to fix it.");
            const vector<int> a = e.get_asymmetric_pads();  // top, bottom, left, right
            Layer *padl = new LPad(p, {a[0], a[3], a[1], a[2]}, 0.0f, n.name + "__asymmetric_padding");
            l = new LConv(padl, wd[0], kernel, strides, "valid", {0, 0, 0, 0}, groups, dilations, use_bias, n.name);
        }
        fill(l->cd->K, n, 1);
        if (use_bias) fill(l->cd->bias, n, 2);
        return l;
    }

    // layers/normalization/batchnorm_onnx.cpp:6-72
    Layer *batchnorm(const NodeP &n) {
        const float eps = n.attr("epsilon") ? n.attr("epsilon")->f : 1e-5f;
        const float momentum = n.attr("momentum") ? n.attr("momentum")->f : 0.9f;
        if (n.input.size() < 5) msg("node " + n.name + ": BatchNormalization needs scale, bias, mean and variance", "ONNX::ImportNet");
        LBatchNorm *l = new LBatchNorm(parent(n), momentum, eps, true, n.name);
        fill(l->bn_g, n, 1);
        fill(l->bn_b, n, 2);
        fill(l->mean, n, 3);
        fill(l->variance, n, 4);
        return l;
    }

    // layers/core/activation_onnx.cpp:183-220
    Layer *softmax(const NodeP &n) {
        Layer *p = parent(n);
        const int nd = (int)p->output->ndim;
        int axis = n.attr("axis") ? (int)n.attr("axis")->i : 1;
        if (axis < 0) axis += nd;
        if (axis < 0 || axis >= nd) msg("The target axis for Softmax is not valid: axis = " + std::to_string(axis), "ONNX::ImportNet");
        if (axis == 0 && nd == 2) axis = 1;
        if (axis == 0) msg("The target axis for Softmax is not valid: axis = " + std::to_string(axis), "ONNX::ImportNet");
        return new LActivation(p, "softmax", {(float)axis}, n.name);
    }

    // layers/pool/maxpool_onnx.cpp:6-128, avgpool_onnx.cpp
    Layer *pool(const NodeP &n, bool is_max) {
        Layer *p = parent(n);
        need_4d(p, n);
        vector<int> kernel, strides, pads;
        for (const AttrP &a : n.attribute) {
            if (a.name == "kernel_shape") kernel = a.int_list();
            else if (a.name == "strides") strides = a.int_list();
            else if (a.name == "pads") {
                pads = a.int_list();
                if (pads.size() == 4) std::swap(pads[1], pads[2]);
            } else if (a.name == "ceil_mode" && a.i)
                info("node " + n.name + ": ceil_mode is ignored, as the reference ignores it (output sizes round down)");
        }
        if (strides.empty()) strides.assign(kernel.size(), 1);
        if (pads.empty()) pads = {0, 0, 0, 0};
        auto make = [&](Layer *from, const vector<int> &pd) -> Layer * {
            if (is_max) return new LMaxPool(from, kernel, strides, pd, n.name);
            return new LAveragePool(from, kernel, strides, pd, n.name);
        };
        try {
            return make(p, pads);
        } catch (const AsymmetricPaddingException &e) {
            info(string("Detected a padding asymmetry in the ") + (is_max ? "MaxPool" : "AveragePool") + " layer \"" + n.name +
                 "\". Going to add an explicit Pad layer before to fix it.");
            const vector<int> a = e.get_asymmetric_pads();
            Layer *padl = new LPad(p, {a[0], a[3], a[1], a[2]}, 0.0f, n.name + "__asymmetric_padding");
            return make(padl, {0, 0, 0, 0});
        }
    }

    // layers/core/dense_onnx.cpp:5-93 (Gemm), layers/merge/matmul_onnx.cpp (a product with an initializer)
    Layer *gemm(const NodeP &n) {
        if (n.attr("alpha") && n.attr("alpha")->f != 1.0f) msg("node " + n.name + ": Gemm with alpha != 1 is not a Dense layer", "ONNX::ImportNet");
        if (n.attr("beta") && n.attr("beta")->f != 1.0f) msg("node " + n.name + ": Gemm with beta != 1 is not a Dense layer", "ONNX::ImportNet");
        if (n.attr("transA") && n.attr("transA")->i) msg("node " + n.name + ": Gemm with transA is not a Dense layer", "ONNX::ImportNet");
        return dense(n, n.attr("transB") ? (int)n.attr("transB")->i : 0);
    }

    Layer *dense(const NodeP &n, int transB) {
        if (n.input.size() < 2 || !layers.count(n.input[0]) || !values.count(n.input[1]))
            msg("node " + n.name + ": only a layer times a constant matrix is a Dense layer", "ONNX::ImportNet");
        Layer *p = layers[n.input[0]];
        const vector<int> &wd = dims[n.input[1]];
        if (wd.size() != 2) msg("node " + n.name + ": the weights of a Dense layer must be a matrix", "ONNX::ImportNet");
        const int in = transB ? wd[1] : wd[0], out = transB ? wd[0] : wd[1];
        if (in != p->output->shape.back()) msg("node " + n.name + ": the weights do not match the input", "ONNX::ImportNet");
        const bool use_bias = n.input.size() > 2;
        LDense *l = new LDense(p, out, use_bias, n.name);
        const vector<float> &w = values[n.input[1]];
        if (w.size() != l->W->size) msg("node " + n.name + ": the weights hold the wrong number of values", "Tensor::copy");
        if (transB) {  // [out, in] in the file, [in, out] in the layer
            for (int o = 0; o < out; o++)
                for (int i = 0; i < in; i++) l->W->ptr[(size_t)i * out + o] = w[(size_t)o * in + i];
        } else {
            memcpy(l->W->ptr, w.data(), w.size() * sizeof(float));
        }
        if (use_bias) fill(l->bias, n, 2);
        return l;
    }

    // layers/merge/add_onnx.cpp:11-143
    Layer *add(const NodeP &n) {
        vector<Layer *> parents;
        const vector<float> *constant = nullptr;
        for (const string &i : n.input) {
            if (layers.count(i)) parents.push_back(layers[i]);
            else if (values.count(i) && constant == nullptr) constant = &values[i];
        }
        if (constant != nullptr) {
            Layer *p = parents.empty() ? nullptr : parents[0];
            if (LConv *c = dynamic_cast<LConv *>(p)) {
                if (constant->size() != c->cd->bias->size) msg("node " + n.name + ": the constant does not match the filters", "ONNX::ImportNet");
                for (size_t i = 0; i < constant->size(); i++)
                    c->cd->bias->ptr[i] = c->cd->use_bias ? c->cd->bias->ptr[i] + (*constant)[i] : (*constant)[i];
                c->cd->use_bias = true;
                return c;
            }
            if (LDense *d = dynamic_cast<LDense *>(p)) {
                if (constant->size() != (size_t)d->ndim) msg("node " + n.name + ": the constant does not match the outputs", "ONNX::ImportNet");
                if (!d->use_bias) {
                    d->bias = new Tensor(vector<int>{d->ndim}, DEV_CPU);
                    d->params.push_back(d->bias);
                    memcpy(d->bias->ptr, constant->data(), constant->size() * sizeof(float));
                    d->use_bias = true;
                } else {
                    for (size_t i = 0; i < constant->size(); i++) d->bias->ptr[i] = (*constant)[i] + d->bias->ptr[i];
                }
                return d;
            }
            if (LBatchNorm *b = dynamic_cast<LBatchNorm *>(p)) {
                if (constant->size() != b->bn_b->size) msg("node " + n.name + ": the constant does not match the channels", "ONNX::ImportNet");
                memcpy(b->bn_b->ptr, constant->data(), constant->size() * sizeof(float));
                return b;
            }
            msg("node " + n.name + ": adding a constant tensor to this layer is outside the forward path this backend implements",
                "ONNX::ImportNet");
        }
        if (parents.size() < 2) msg("Error in Add node " + n.name + ". Unable to process its inputs", "ONNX::ImportNet");
        return new LAdd(parents, n.name);
    }

    // layers/merge/concat_onnx.cpp:5-49
    Layer *concat(const NodeP &n) {
        vector<Layer *> parents;
        for (size_t i = 0; i < n.input.size(); i++) parents.push_back(parent(n, i));
        int axis = n.attr("axis") ? (int)n.attr("axis")->i : 1;
        if (axis < 0) axis += (int)parents[0]->output->ndim;
        if (axis == 0) msg("Error in Concat layer " + n.name + ". Concat by the dimension 0 is not allowed.", "ONNX::ImportNet");
        return new LConcat(parents, (unsigned)(axis - 1), n.name);
    }

    void nearest_only(const NodeP &n) {
        const string mode = n.attr("mode") ? n.attr("mode")->s : "nearest";
        if (mode != "nearest") msg("In Resize operator, the mode \"" + mode + "\" is not supported. It must be \"nearest\".", "ONNX::ImportNet");
    }

    Layer *upsampled(Layer *p, const NodeP &n, int th, int tw) {
        const int h = p->output->shape[2], w = p->output->shape[3];
        if (th < h || tw < w || th % h || tw % w)
            msg("node " + n.name + ": only whole-number upscaling is on this backend's path", "ONNX::ImportNet");
        return new LResize(p, {th, tw}, n.name);
    }

    // layers/conv/upsampling2D_onnx.cpp:5-72
    Layer *upsample(const NodeP &n) {
        Layer *p = parent(n);
        need_4d(p, n);
        nearest_only(n);
        vector<float> scales;
        if (n.input.size() > 1 && values.count(n.input[1])) scales = values[n.input[1]];
        else if (n.attr("scales")) scales = n.attr("scales")->floats;  // opset 7 keeps them in an attribute
        if (scales.size() != 4) msg("Error in node " + n.name + ". Unexpected number of scale values, expected 4.", "ONNX::ImportNet");
        return upsampled(p, n, p->output->shape[2] * (int)scales[2], p->output->shape[3] * (int)scales[3]);
    }

    // layers/core/resize_onnx.cpp:5-62; inputs by position: X, roi, scales, sizes (an absent one is an empty name)
    Layer *resize(const NodeP &n) {
        Layer *p = parent(n);
        need_4d(p, n);
        nearest_only(n);
        vector<string> pos = n.positional;
        pos.resize(4);
        const int h = p->output->shape[2], w = p->output->shape[3];
        if (values.count(pos[3]) && values[pos[3]].size() == 4) return upsampled(p, n, (int)values[pos[3]][2], (int)values[pos[3]][3]);
        const string &sc = values.count(pos[2]) && values[pos[2]].size() == 4 ? pos[2] : pos[1];
        if (!values.count(sc) || values[sc].size() != 4) msg("node " + n.name + ": neither sizes nor scales are constants", "ONNX::ImportNet");
        return upsampled(p, n, (int)(h * values[sc][2]), (int)(w * values[sc][3]));
    }

    // layers/da/pad_onnx.cpp:5-110
    Layer *pad(const NodeP &n) {
        Layer *p = parent(n);
        const string mode = n.attr("mode") ? n.attr("mode")->s : "constant";
        if (mode != "constant")
            msg("Error importing layer " + n.name + ". Only \"constant\" mode is supported (passed \"" + mode + "\").", "ONNX::ImportNet");
        float constant = n.attr("value") ? n.attr("value")->f : 0.0f;
        vector<int> pads;
        if (n.attr("pads")) {
            pads = n.attr("pads")->int_list();
        } else {
            if (n.input.size() < 2 || !values.count(n.input[1]))
                msg("Error importing layer " + n.name + ". The padding values are not constants.", "ONNX::ImportNet");
            for (float v : values[n.input[1]]) pads.push_back((int)v);
            if (n.input.size() > 2 && values.count(n.input[2])) {
                if (values[n.input[2]].size() != 1)
                    msg("Unexpected error importing layer " + n.name + ". The number of constant values is not 1", "ONNX::ImportNet");
                constant = values[n.input[2]][0];
            }
        }
        if (pads.size() != 8)
            msg("Error importing layer " + n.name + ". The expected number of padding values is 8, got " + std::to_string(pads.size()) + ".",
                "ONNX::ImportNet");
        if (pads[0] || pads[1] || pads[4] || pads[5])
            msg("Error importing layer " + n.name + ". Padding the batch or the channels is not supported.", "ONNX::ImportNet");
        // (batch_b, ch_b, h_b, w_b, batch_e, ch_e, h_e, w_e) -> (top, right, bottom, left)
        return new LPad(p, {pads[2], pads[7], pads[6], pads[3]}, constant, n.name);
    }

    // layers/core/reshape_onnx.cpp:5-68
    Layer *reshape(const NodeP &n) {
        if (n.input.size() < 2 || !values.count(n.input[1])) msg("node " + n.name + ": the target shape is not a constant", "ONNX::ImportNet");
        vector<int> shape;
        for (float v : values[n.input[1]]) shape.push_back((int)v);
        if (layers.count(n.input[0])) {
            Layer *p = layers[n.input[0]];
            for (size_t i = 0; i < shape.size(); i++)
                if (shape[i] == 0 && i < p->output->shape.size()) shape[i] = p->output->shape[i];  // 0 copies the input dimension
            if (shape.empty()) msg("node " + n.name + ": empty target shape", "ONNX::ImportNet");
            shape[0] = 1;  // the first entry is the batch
            return new LReshape(p, shape, n.name);
        }
        for (const string &o : n.output) {  // a reshaped parameter stays a parameter
            values[o] = values[n.input[0]];
            dims[o] = shape;
        }
        return nullptr;
    }
};

Net *import_bytes(const void *data, size_t size, const vector<int> &input_shape) {
    Span s;
    s.p = static_cast<const uint8_t *>(data);
    s.n = size;
    try {
        GraphP graph(s);
        return Importer(graph, input_shape).run();
    } catch (const ParseError &e) {
        msg(string("Failed to parse model: ") + e.what(), "ONNX::ImportNet");
    }
    return nullptr;
}

// ---------------------------------------------------------------- writing
class Writer {
  public:
    string out;
    void varint(uint64_t v) {
        while (v >= 0x80) {
            out.push_back((char)((v & 0x7F) | 0x80));
            v >>= 7;
        }
        out.push_back((char)v);
    }
    void key(int field, int wire) { varint(((uint64_t)field << 3) | (uint64_t)wire); }
    void bytes(int field, const string &data) {
        key(field, 2);
        varint(data.size());
        out += data;
    }
    void integer(int field, int64_t v) {
        key(field, 0);
        varint((uint64_t)v);
    }
    void real(int field, float v) {
        key(field, 5);
        out.append(reinterpret_cast<const char *>(&v), 4);
    }
};

// AttributeProto.AttributeType: FLOAT 1, INT 2, STRING 3, TENSOR 4, INTS 7
string attr_ints(const string &name, const vector<int> &v) {
    Writer w, packed;
    for (int x : v) packed.varint((uint64_t)(int64_t)x);
    w.bytes(1, name);
    w.bytes(8, packed.out);
    w.integer(20, 7);
    return w.out;
}
string attr_int(const string &name, int64_t v) {
    Writer w;
    w.bytes(1, name);
    w.integer(3, v);
    w.integer(20, 2);
    return w.out;
}
string attr_float(const string &name, float v) {
    Writer w;
    w.bytes(1, name);
    w.real(2, v);
    w.integer(20, 1);
    return w.out;
}
string attr_string(const string &name, const string &v) {
    Writer w;
    w.bytes(1, name);
    w.bytes(4, v);
    w.integer(20, 3);
    return w.out;
}
string attr_tensor(const string &name, const string &tensor) {
    Writer w;
    w.bytes(1, name);
    w.bytes(5, tensor);
    w.integer(20, 4);
    return w.out;
}

// float_data / int64_data, not raw_data: what the reference's exporter writes (e.g. conv_onnx.cpp:283-297)
string tensor_floats(const string &name, const vector<int> &shape, const float *data, size_t count) {
    Writer w, d;
    for (int x : shape) d.varint((uint64_t)x);
    if (!shape.empty()) w.bytes(1, d.out);
    w.integer(2, FLOAT);
    w.bytes(4, string(reinterpret_cast<const char *>(data), count * sizeof(float)));
    w.bytes(8, name);
    return w.out;
}
string tensor_of(const string &name, Tensor *t) {
    Tensor host(t->getShape(), DEV_CPU);
    Tensor::copy(t, &host);
    return tensor_floats(name, host.shape, host.ptr, host.size);
}
string tensor_int64(const string &name, const vector<int64_t> &v) {
    Writer w, d, p;
    d.varint(v.size());
    w.bytes(1, d.out);
    w.integer(2, INT64);
    for (int64_t x : v) p.varint((uint64_t)x);
    w.bytes(7, p.out);
    w.bytes(8, name);
    return w.out;
}

string node(const string &op, const string &name, const vector<string> &inputs, const vector<string> &outputs,
            const vector<string> &attrs = {}) {
    Writer w;
    for (const string &i : inputs) w.bytes(1, i);
    for (const string &o : outputs) w.bytes(2, o);
    w.bytes(3, name);
    w.bytes(4, op);
    for (const string &a : attrs) w.bytes(5, a);
    return w.out;
}

string value_info(const string &name, const vector<int> &shape) {
    Writer dims;
    {
        Writer d;
        d.bytes(2, "batch");
        dims.bytes(1, d.out);
    }
    for (size_t i = 1; i < shape.size(); i++) {
        Writer d;
        d.integer(1, shape[i]);
        dims.bytes(1, d.out);
    }
    Writer tt, ty, vi;
    tt.integer(1, FLOAT);
    tt.bytes(2, dims.out);
    ty.bytes(1, tt.out);
    vi.bytes(1, name);
    vi.bytes(2, ty.out);
    return vi.out;
}

}  // namespace

// ---------------------------------------------------------------- entry points
Net *import_net_from_onnx_file(const string &path, const vector<int> &input_shape, int) {
    std::ifstream in(path, std::ios::in | std::ios::binary);
    if (!in.good()) msg("The specified path does not exist: " + path, "ONNX::ImportNet");
    std::stringstream ss;
    ss << in.rdbuf();
    const string data = ss.str();
    return import_bytes(data.data(), data.size(), input_shape);
}

Net *import_net_from_onnx_pointer(const void *serialized_model, size_t size, int) { return import_bytes(serialized_model, size, {}); }

Net *import_net_from_onnx_string(const string *model_string, int) { return import_bytes(model_string->data(), model_string->size(), {}); }

// build_onnx_model / set_graph (export_helpers.cpp:8-120): producer "EDDL" 1.0, opset 11, inputs and outputs
// with a symbolic batch, one node per layer in layer order, values named after the layers, parameters as
// initializers <layer>_W, _b, _scale, _bias, _mean, _variance.
string serialize_net_to_onnx_string(Net *net) {
    vector<string> nodes, inits;
    for (Layer *l : net->layers) {
        vector<string> ins;
        for (Layer *p : l->parent) ins.push_back(p->name);
        if (dynamic_cast<LInput *>(l)) continue;
        if (LConv *c = dynamic_cast<LConv *>(l)) {
            ConvolDescriptor *cd = c->cd;
            ins.push_back(l->name + "_W");
            inits.push_back(tensor_of(l->name + "_W", cd->K));
            if (cd->use_bias) {
                ins.push_back(l->name + "_b");
                inits.push_back(tensor_of(l->name + "_b", cd->bias));
            }
            nodes.push_back(node("Conv", l->name, ins, {l->name},
                                 {attr_ints("dilations", cd->dilation_rate), attr_int("group", cd->groups),
                                  attr_ints("kernel_shape", {cd->kr, cd->kc}),
                                  attr_ints("pads", {cd->padrt, cd->padcl, cd->padrb, cd->padcr}), attr_ints("strides", {cd->sr, cd->sc})}));
        } else if (LBatchNorm *b = dynamic_cast<LBatchNorm *>(l)) {
            const int C = b->input->shape[1];
            const vector<float> ones(C, 1.0f), zeros(C, 0.0f);
            ins.push_back(l->name + "_scale");
            inits.push_back(b->affine ? tensor_of(l->name + "_scale", b->bn_g) : tensor_floats(l->name + "_scale", {C}, ones.data(), C));
            ins.push_back(l->name + "_bias");
            inits.push_back(b->affine ? tensor_of(l->name + "_bias", b->bn_b) : tensor_floats(l->name + "_bias", {C}, zeros.data(), C));
            ins.push_back(l->name + "_mean");
            inits.push_back(tensor_of(l->name + "_mean", b->mean));
            ins.push_back(l->name + "_variance");
            inits.push_back(tensor_of(l->name + "_variance", b->variance));
            nodes.push_back(node("BatchNormalization", l->name, ins, {l->name},
                                 {attr_float("epsilon", b->epsilon), attr_float("momentum", b->momentum)}));
        } else if (LActivation *a = dynamic_cast<LActivation *>(l)) {
            if (a->act == "relu") nodes.push_back(node("Relu", l->name, ins, {l->name}));
            else if (a->act == "sigmoid") nodes.push_back(node("Sigmoid", l->name, ins, {l->name}));
            else nodes.push_back(node("Softmax", l->name, ins, {l->name}, {attr_int("axis", (int)a->act_params[0])}));
        } else if (LPool *pl = dynamic_cast<LPool *>(l)) {
            PoolDescriptor *pd = pl->pd;
            nodes.push_back(node(dynamic_cast<LMaxPool *>(l) ? "MaxPool" : "AveragePool", l->name, ins, {l->name},
                                 {attr_ints("kernel_shape", {pd->kr, pd->kc}),
                                  attr_ints("pads", {pd->padrt, pd->padcl, pd->padrb, pd->padcr}), attr_ints("strides", {pd->sr, pd->sc})}));
        } else if (LResize *r = dynamic_cast<LResize *>(l)) {
            const float roi[8] = {0, 0, 0, 0, 1, 1, 1, 1};
            const float scales[4] = {1.0f, 1.0f, (float)(r->new_shape[0] / r->input->shape[2]), (float)(r->new_shape[1] / r->input->shape[3])};
            inits.push_back(tensor_floats(l->name + "_roi", {8}, roi, 8));
            inits.push_back(tensor_floats(l->name + "_scales", {4}, scales, 4));
            ins.push_back(l->name + "_roi");
            ins.push_back(l->name + "_scales");
            nodes.push_back(node("Resize", l->name, ins, {l->name},
                                 {attr_string("coordinate_transformation_mode", "asymmetric"), attr_string("mode", "nearest")}));
        } else if (LConcat *cc = dynamic_cast<LConcat *>(l)) {
            nodes.push_back(node("Concat", l->name, ins, {l->name}, {attr_int("axis", (int)cc->axis + 1)}));
        } else if (dynamic_cast<LAdd *>(l)) {
            nodes.push_back(node("Add", l->name, ins, {l->name}));
        } else if (dynamic_cast<LSum *>(l)) {
            nodes.push_back(node("Sum", l->name, ins, {l->name}));
        } else if (LPad *pd = dynamic_cast<LPad *>(l)) {
            inits.push_back(tensor_int64(l->name + "_pads", {0, 0, pd->padding[0], pd->padding[3], 0, 0, pd->padding[2], pd->padding[1]}));
            inits.push_back(tensor_floats(l->name + "_value", {}, &pd->constant, 1));
            ins.push_back(l->name + "_pads");
            ins.push_back(l->name + "_value");
            nodes.push_back(node("Pad", l->name, ins, {l->name}, {attr_string("mode", "constant")}));
        } else if (LReshape *rs = dynamic_cast<LReshape *>(l)) {
            vector<int64_t> target(rs->ls.begin(), rs->ls.end());
            target[0] = -1;
            nodes.push_back(node("Constant", "", {}, {l->name + "_target_shape"}, {attr_tensor("value", tensor_int64("const_tensor", target))}));
            ins.push_back(l->name + "_target_shape");
            nodes.push_back(node("Reshape", l->name, ins, {l->name}));
        } else if (LDense *d = dynamic_cast<LDense *>(l)) {
            ins.push_back(l->name + "_W");
            inits.push_back(tensor_of(l->name + "_W", d->W));
            if (d->use_bias) {
                ins.push_back(l->name + "_b");
                inits.push_back(tensor_of(l->name + "_b", d->bias));
            }
            if (d->input->ndim == 2) {
                nodes.push_back(node("Gemm", l->name, ins, {l->name},
                                     {attr_float("alpha", 1.0f), attr_float("beta", 1.0f), attr_int("transA", 0), attr_int("transB", 0)}));
            } else {  // build_dense_with_matmul_node: MatMul, then Add of the bias
                const string mm = d->use_bias ? l->name + "_MatMul" : l->name;
                nodes.push_back(node("MatMul", mm, {ins[0], ins[1]}, {mm}));
                if (d->use_bias) nodes.push_back(node("Add", l->name, {mm, ins[2]}, {l->name}));
            }
        } else {
            msg("layer " + l->name + " has no ONNX form here", "ONNX::ExportNet");
        }
    }
    Writer graph;
    for (const string &n : nodes) graph.bytes(1, n);
    graph.bytes(2, "Computational Graph");
    for (const string &t : inits) graph.bytes(5, t);
    for (Layer *l : net->layers)
        if (dynamic_cast<LInput *>(l)) graph.bytes(11, value_info(l->name, l->output->shape));
    for (Layer *l : net->lout) graph.bytes(12, value_info(l->name, l->output->shape));
    Writer opset, model;
    opset.integer(2, 11);
    model.integer(1, 6);
    model.bytes(2, "EDDL");
    model.bytes(3, "1.0");
    model.bytes(7, graph.out);
    model.bytes(8, opset.out);
    return model.out;
}

void save_net_to_onnx_file(Net *net, const string &path) {
    const string data = serialize_net_to_onnx_string(net);
    std::ofstream ofs(path, std::ios::out | std::ios::binary);
    ofs.write(data.data(), (std::streamsize)data.size());
    if (!ofs.good()) msg("cannot write " + path, "ONNX::ExportNet");
}

}  // namespace eddl_hip
