// Layers, Net and the eddl:: model-building API of the CNN forward path, in C++, above
// eddl_hip_host.h (Tensor, descriptors, tensorNN).  Each class keeps the name, the constructor
// arguments, the parameter order and the forward() call of its reference counterpart:
//   Layer              include/eddl/layers/layer.h:32-140, src/layers/layer.cpp
//   LInput             src/layers/core/layer_input.cpp
//   LConv              src/layers/conv/layer_conv2D.cpp:24-62,91-93
//   LBatchNorm         src/layers/normalization/layer_batchnorm.cpp:26-135,186-262
//   LActivation        src/layers/core/layer_activation.cpp:21-33,168-196   (relu, sigmoid, softmax)
//   LMaxPool           src/layers/pool/layer_maxpool.cpp:29-64
//   LAveragePool       src/layers/pool/layer_avgpool2D.cpp:29-58
//   LResize            src/layers/core/layer_resize.cpp:22-47               (UpSampling2D)
//   LConcat            src/layers/merge/layer_concat.cpp:25-94
//   LAdd, LSum         src/layers/merge/layer_add.cpp:25-64, src/layers/operators/layer_sum.cpp:33-78
//   LPad               src/layers/da/layer_pad.cpp:23-46
//   LReshape           src/layers/core/layer_reshape.cpp:22-135
//   LDense             src/layers/core/layer_dense.cpp:25-73
//   Net                src/net/net.cpp:77-114,231-258,411-449; src/net/net_build.cpp:34-70,414-465;
//                      src/net/net_api.cpp:266-298,1436-1457
//   eddl:: functions   include/eddl/apis/eddl.h, src/apis/eddl.cpp
// Differences that follow from this being a forward-only device backend: layers are created on
// the host with batch size 1, as in the reference, but nothing computes there; build() with a
// CS_HIP computing service moves every tensor to the GPU (the reference clones the net per
// device instead) and forward() runs the layers on it.  Training, losses, optimisers and
// metrics are absent: build() takes only the computing service.
#pragma once
#include <stdexcept>

#include "eddl_hip_host.h"

namespace eddl_hip {

constexpr int TRMODE = 1;  // include/eddl/layers/layer.h:23-24
constexpr int TSMODE = 0;

class Net;

class Layer {
  public:
    string name;
    Tensor *input = nullptr;
    Tensor *output = nullptr;
    vector<Tensor *> params;
    vector<Layer *> parent, child;
    Net *net = nullptr;
    int mode = TSMODE;
    int dev = DEV_CPU;
    int lin = 0, lout = 0;

    Layer(const string &name, const string &default_prefix);
    virtual ~Layer();
    virtual void forward() = 0;
    virtual void resize(int batch);      // default: the output follows the batch
    virtual void toGPU(int device);      // default: output and parameters move
    virtual void initialize() {}  // parameters at build(init_weights = true), drawn on the device
    virtual string kind() const = 0;
    vector<int> getShape() const { return output->getShape(); }
    void addchild(Layer *l);
    void addparent(Layer *l);
    void setmode(int m) { mode = m; }

  protected:
    vector<Tensor *> extra;  // further batch-shaped tensors the layer owns (indices, side outputs)
    vector<Tensor *> fixed;  // further tensors that do not depend on the batch (statistics scratch)
    static int total_layers;
};

// thrown like the reference's (src/layers/conv/layer_conv2D.cpp:57-61, include/eddl/utils.h)
class AsymmetricPaddingException : public std::runtime_error {
  public:
    vector<int> asymmetric_pads;
    AsymmetricPaddingException(const string &msg, const vector<int> &pads) : std::runtime_error(msg), asymmetric_pads(pads) {}
    vector<int> get_asymmetric_pads() const { return asymmetric_pads; }
};

class LInput : public Layer {
  public:
    LInput(Tensor *in, string name);
    void forward() override {}
    string kind() const override { return "input"; }
};

class LConv : public Layer {
  public:
    ConvolDescriptor *cd;
    LConv(Layer *parent, int filters, const vector<int> &kernel_size, const vector<int> &strides, string padding, const vector<int> &pads,
          int groups, const vector<int> &dilation_rate, bool use_bias, string name);
    ~LConv() override;
    void forward() override;
    void resize(int batch) override;
    void initialize() override;
    string kind() const override { return "conv2d"; }
};

class LBatchNorm : public Layer {
  public:
    float momentum, epsilon;
    bool affine;
    Tensor *mean, *variance, *bn_mean, *bn_var, *bn_g = nullptr, *bn_b = nullptr, *opa;
    LBatchNorm(Layer *parent, float momentum, float epsilon, bool affine, string name);
    void forward() override;
    void initialize() override;
    string kind() const override { return "batchnorm"; }
};

class LActivation : public Layer {
  public:
    string act;
    vector<float> act_params;
    LActivation(Layer *parent, string act, vector<float> params, string name);
    void forward() override;
    string kind() const override { return act; }
};

class LPool : public Layer {
  public:
    PoolDescriptor *pd;
    LPool(Layer *parent, PoolDescriptor *pd, const string &name, const string &prefix);
    ~LPool() override;
    void resize(int batch) override;
};

class LMaxPool : public LPool {
  public:
    LMaxPool(Layer *parent, const vector<int> &pool_size, const vector<int> &strides, const string &padding, string name);
    LMaxPool(Layer *parent, const vector<int> &pool_size, const vector<int> &strides, const vector<int> &padding, string name);
    void forward() override;
    void resize(int batch) override;
    void toGPU(int device) override;
    string kind() const override { return "maxpool2d"; }

  private:
    void make_indices();
};

class LAveragePool : public LPool {
  public:
    LAveragePool(Layer *parent, const vector<int> &pool_size, const vector<int> &strides, const string &padding, string name);
    LAveragePool(Layer *parent, const vector<int> &pool_size, const vector<int> &strides, const vector<int> &padding, string name);
    void forward() override;
    string kind() const override { return "avgpool2d"; }
};

class LResize : public Layer {
  public:
    vector<int> new_shape;  // target height, width
    LResize(Layer *parent, vector<int> new_shape, string name);
    void forward() override;
    string kind() const override { return "resize"; }
};

class LConcat : public Layer {
  public:
    unsigned int axis;  // batch not included
    LConcat(vector<Layer *> parent, unsigned int axis, string name);
    void forward() override;
    string kind() const override { return "concat"; }
};

class LAdd : public Layer {
  public:
    LAdd(vector<Layer *> parent, string name);
    void forward() override;
    string kind() const override { return "add_n"; }
};

class LSum : public Layer {
  public:
    LSum(Layer *l1, Layer *l2, string name);
    void forward() override;
    string kind() const override { return "sum"; }
};

class LPad : public Layer {
  public:
    vector<int> padding;  // top, right, bottom, left
    float constant;
    LPad(Layer *parent, vector<int> padding, float constant, string name);
    void forward() override;
    void resize(int batch) override;
    void toGPU(int device) override;
    string kind() const override { return "pad"; }
};

class LReshape : public Layer {
  public:
    vector<int> ls;
    LReshape(Layer *parent, vector<int> shape, string name);
    ~LReshape() override;
    void forward() override {}
    void resize(int batch) override;
    void toGPU(int device) override;
    string kind() const override { return "reshape"; }
};

class LDense : public Layer {
  public:
    int ndim;
    bool use_bias;
    Tensor *W, *bias = nullptr;
    LDense(Layer *parent, int ndim, bool use_bias, string name);
    void forward() override;
    void initialize() override;
    string kind() const override { return "dense"; }
};

// Computing service: which GPUs run the net (src/net/compserv.cpp:34-56).  local_gpus is the
// reference's mask: entry i set = use GPU i.
struct CompServ {
    string type = "hip";
    vector<int> local_gpus;
    int lsb = 1;
    string mem = "full_mem";
};

// One step of a fused inference plan (Net::fuse): either one layer's forward(), or a convolution /
// dense layer together with the layers that follow it and are computed in the same kernel.
struct FusedStep {
    Layer *first = nullptr;     // the layer the step starts at
    Layer *last = nullptr;      // the layer whose output tensor the step writes
    Layer *src = nullptr;       // conv chains: the layer whose output is read (a folded zero pad's parent)
    Layer *src2 = nullptr;      // conv chains: a folded channel Concat's second parent (src is then its first)
    LBatchNorm *bn = nullptr;   // conv chains: inference batch norm applied to the sums
    Layer *res = nullptr;       // conv chains: the other operand of a residual LSum
    bool relu = false;
    int pad_top = 0, pad_left = 0;
    int up_h = 1, up_w = 1;     // conv chains: whole factors of a folded nearest UpSampling2D (src is then its parent)
    bool chain = false;         // false: first->forward()
    LPool *pool = nullptr;      // conv chains: a 2x2, stride-2, unpadded LMaxPool of last's output computed by the same call
    bool keep = true;           // conv chains with a pool: some other layer (or the caller) reads last's output as well
};

class Net {
  public:
    string name = "model";
    vector<Layer *> lin, lout, layers;  // layers: the reference's forward order
    int batch_size = 1;
    int dev = DEV_CPU;
    CompServ *cs = nullptr;

    Net(const vector<Layer *> &in, const vector<Layer *> &out);
    ~Net();
    void build(CompServ *cs, bool init_weights = true);
    void resize(int batch);
    void setmode(int m);
    void forward(const vector<Tensor *> &in);
    void forward();
    vector<Tensor *> predict(const vector<Tensor *> &in);
    void save(const string &filename, const string &format = "bin");
    void load(const string &filename, const string &format = "bin");
    string summary(bool print_stdout = true);
    // Parameters per layer, in `layers` order (src/net/net_api.cpp:199-260).  The tensors handed out are
    // host copies owned by the caller (the reference's deepcopy = true; without it the reference hands
    // out its own host-side tensors, which this device-resident net does not keep).
    vector<vector<Tensor *>> get_parameters(bool deepcopy = true);
    void set_parameters(const vector<vector<Tensor *>> &params);
    Layer *getLayer(const string &name);

    // Inference plan with the layer chains conv [+ batchnorm] [+ sum] [+ relu], zero pad + conv and
    // dense + relu each computed by one kernel, and the repacked filters of every convolution kept
    // between calls.  No counterpart in the reference (whose forward() always walks `layers`);
    // results are the ones of the layer-by-layer walk, bit for bit.  Layers inside a chain leave
    // their own output tensors unwritten (is_fused_away tells which); batch-norm layers inside a
    // chain do not update their side outputs.  forward() queues the plan without waiting between
    // steps and waits once at the end.
    void fuse();
    bool is_fused_away(const Layer *l) const;
    vector<FusedStep> plan;  // empty until fuse()

  private:
    void run_step(const FusedStep &s);
    vector<const Layer *> fused_away;
};

namespace eddl {

typedef Layer *layer;
typedef Net *model;
typedef vector<Layer *> vlayer;
typedef vector<Tensor *> vtensor;
typedef CompServ *compserv;

model Model(vlayer in, vlayer out);
void setName(model m, string name);
// one GPU: exactly one entry of g may be set
compserv CS_HIP(const vector<int> &g, const string &mem = "full_mem");
compserv CS_GPU(const vector<int> &g, const string &mem = "full_mem");  // the reference's spelling, same service
void build(model net, compserv cs, bool init_weights = true);
void fuse(model net);  // Net::fuse: the fused inference plan (this backend's addition)
void show_profile();   // src/apis/eddl.cpp:291-297: the host wall-clock profile of forward and of the functions it called
void reset_profile();
void set_mode(model net, int mode);
void summary(model m);
void load(model m, const string &fname, const string &format = "bin");
void save(model m, const string &fname, const string &format = "bin");
vlayer forward(model m, vtensor in);
vtensor predict(model m, const vtensor &in);
Tensor *getOutput(layer l1);  // a host copy, owned by the caller
vector<vtensor> get_parameters(model net, bool deepcopy = true);
void set_parameters(model net, const vector<vtensor> &params);
layer getLayer(model net, const string &name);
vlayer getOut(model net);
vtensor getParams(layer l1);  // host copies, owned by the caller

layer Input(const vector<int> &shape, string name = "");
layer Conv2D(layer parent, int filters, const vector<int> &kernel_size, const vector<int> &strides = {1, 1}, string padding = "same",
             bool use_bias = true, int groups = 1, const vector<int> &dilation_rate = {1, 1}, string name = "");
layer Dense(layer parent, int ndim, bool use_bias = true, string name = "");
layer Activation(layer parent, string activation, vector<float> params = {}, string name = "");
layer ReLu(layer parent, string name = "");
layer Sigmoid(layer parent, string name = "");
layer Softmax(layer parent, int axis = -1, string name = "");
layer BatchNormalization(layer parent, float momentum = 0.99f, float epsilon = 0.001f, bool affine = true, string name = "");
layer BatchNormalization(layer parent, bool affine, float momentum = 0.99f, float epsilon = 0.001f, string name = "");
layer MaxPool2D(layer parent, vector<int> pool_size = {2, 2}, vector<int> strides = {2, 2}, string padding = "none", string name = "");
layer AveragePool2D(layer parent, vector<int> pool_size = {2, 2}, vector<int> strides = {2, 2}, string padding = "none",
                    string name = "");
layer AvgPool2D(layer parent, vector<int> pool_size = {2, 2}, vector<int> strides = {2, 2}, string padding = "none", string name = "");
layer GlobalAveragePool2D(layer parent, string name = "");
layer UpSampling2D(layer parent, const vector<int> &size, string interpolation = "nearest", string name = "");
layer Concat(const vector<layer> &layers, unsigned int axis = 0, string name = "");
layer Add(const vector<layer> &layers, string name = "");
layer Add(layer l1, layer l2);
layer Pad(layer parent, vector<int> padding, float constant = 0.0f, string name = "");
layer Reshape(layer parent, const vector<int> &shape, string name = "");
layer Flatten(layer parent, string name = "");

}  // namespace eddl
}  // namespace eddl_hip
