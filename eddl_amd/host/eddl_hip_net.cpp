// Layers, Net and the eddl:: API of the CNN forward path (see eddl_hip_net.h for what each class mirrors).
#include "eddl_hip_net.h"

#include <cmath>
#include <cstdint>
#include <cstring>
#include <fstream>
#include <iomanip>
#include <iostream>
#include <set>
#include <sstream>

#include "../../include/eddlhip.h"

namespace eddl_hip {

// ---------------------------------------------------------------- Layer
int Layer::total_layers = 0;

Layer::Layer(const string &n, const string &default_prefix) : name(n) {
    if (name.empty()) name = default_prefix + std::to_string(++total_layers);
}

Layer::~Layer() {
    delete output;
    for (Tensor *t : params) delete t;
    for (Tensor *t : extra) delete t;
    for (Tensor *t : fixed) delete t;
}

void Layer::addchild(Layer *l) {
    child.push_back(l);
    lout++;
}

void Layer::addparent(Layer *l) {
    parent.push_back(l);
    lin++;
}

void Layer::resize(int batch) {
    output->resize(batch);
    for (Tensor *t : extra) t->resize(batch);
}

void Layer::toGPU(int device) {
    dev = device;
    output->toGPU(device);
    for (Tensor *t : params) t->toGPU(device);
    for (Tensor *t : extra) t->toGPU(device);
    for (Tensor *t : fixed) t->toGPU(device);
}

// Parameter initialisation of build(init_weights = true): Glorot-uniform filters and weights, zero biases (the
// reference's defaults: LConv::initialize, src/layers/conv/layer_conv2D.cpp:109-112, with IGlorotUniform::apply,
// src/initializers/initializer_glorot_uniform.cpp:35-60).  It runs on the DEVICE tensors, through the same calls the
// reference's initialiser makes on the device copy of a net (Net::split -> make_graph -> do_initialize,
// src/net/net_build.cpp:235-237,401): fill_rand_signed_uniform_(1.0) then mult_(limit).
namespace {
void glorot_uniform(Tensor *params) {
    int fin, fout;
    if (params->ndim == 4) {  // (output_depth, input_depth, kr, kc)
        const int rf = params->shape[2] * params->shape[3];
        fin = rf * params->shape[1];
        fout = rf * params->shape[0];
    } else if (params->ndim == 2) {
        fin = params->shape[0];
        fout = params->shape[1];
    } else {
        fin = fout = params->shape[0];
    }
    params->fill_rand_signed_uniform_(1.0f);
    params->mult_(std::sqrt(6.0f / (float)(fin + fout)));
}
}  // namespace

// ---------------------------------------------------------------- LInput
LInput::LInput(Tensor *in, string n) : Layer(n, "input") {
    input = output = in;
}

// ---------------------------------------------------------------- LConv
LConv::LConv(Layer *p, int filters, const vector<int> &kernel_size, const vector<int> &strides, string padding, const vector<int> &pads,
             int groups, const vector<int> &dilation_rate, bool use_bias, string n)
    : Layer(n, "conv2d") {
    if (p->output->ndim != 4) msg("LConv only works over 4D tensors", "LConv::LConv");
    cd = new ConvolDescriptor(filters, kernel_size, strides, padding, pads, groups, dilation_rate, use_bias, 0);
    input = p->output;
    cd->build(input);
    output = cd->O;
    params.push_back(cd->K);
    params.push_back(cd->bias);
    if (cd->pads[0] != cd->pads[1] || cd->pads[2] != cd->pads[3]) {
        string text = "In layer " + name + ": Padding asymmetry detected (top=" + std::to_string(cd->pads[0]) +
                      ", bottom=" + std::to_string(cd->pads[1]) + ", left=" + std::to_string(cd->pads[2]) +
                      ", right=" + std::to_string(cd->pads[3]) +
                      "). The padding asymmetry is not allowed in a Conv layer, we suggest you to use an explicit padding layer "
                      "before this layer to fix the asymmetry.";
        vector<int> asym = cd->pads;
        delete cd;
        cd = nullptr;
        throw AsymmetricPaddingException(text, asym);  // the base destructor releases the tensors
    }
    p->addchild(this);
    addparent(p);
}

LConv::~LConv() { delete cd; }

void LConv::forward() { tensorNN::Conv2D(cd); }

void LConv::resize(int batch) {
    cd->I = input;
    cd->resize(batch);
}

void LConv::initialize() {
    glorot_uniform(cd->K);
    cd->bias->fill_(0.0f);
}

// ---------------------------------------------------------------- LBatchNorm
LBatchNorm::LBatchNorm(Layer *p, float mom, float eps, bool aff, string n)
    : Layer(n, "batchnorm"), momentum(mom), epsilon(eps), affine(aff) {
    input = p->output;
    if (input->ndim != 2 && input->ndim != 4)
        std::cerr << "LBatchNorm only works over 1D or 2D tensors, however, we do not exit here and allow 3D tensors\n";
    const vector<int> shape = {input->shape[1]};
    output = new Tensor(input->getShape(), DEV_CPU);
    opa = Tensor::zeros(input->getShape(), DEV_CPU);
    extra.push_back(opa);
    mean = Tensor::zeros(shape, DEV_CPU);
    variance = Tensor::full(shape, momentum > 0.0f ? 0.0f : 1.0f, DEV_CPU);
    bn_mean = new Tensor(shape, DEV_CPU);
    bn_var = new Tensor(shape, DEV_CPU);
    fixed.push_back(bn_mean);
    fixed.push_back(bn_var);
    if (affine) {
        bn_g = Tensor::ones(shape, DEV_CPU);
        bn_b = Tensor::zeros(shape, DEV_CPU);
        params.push_back(bn_g);
        params.push_back(bn_b);
    }
    params.push_back(mean);
    params.push_back(variance);
    p->addchild(this);
    addparent(p);
}

void LBatchNorm::forward() {
    tensorNN::BatchNormForward(input, output, opa, mean, variance, affine ? bn_g : nullptr, affine ? bn_b : nullptr, bn_mean, bn_var,
                               mode == TRMODE, epsilon, momentum);
}

void LBatchNorm::initialize() {
    if (affine) {
        bn_g->fill_(1.0f);
        bn_b->fill_(0.0f);
    }
}

// ---------------------------------------------------------------- LActivation
LActivation::LActivation(Layer *p, string a, vector<float> prm, string n) : Layer(n, a), act(a), act_params(prm) {
    if (act != "relu" && act != "sigmoid" && act != "softmax")
        msg("activation " + act + " is outside the forward path this backend implements", "LActivation::LActivation");
    input = p->output;
    output = new Tensor(input->shape, DEV_CPU);
    if (act == "softmax") {
        if (act_params.empty()) {
            act_params.push_back(-1);
            std::cerr << "No axis for 'softmax' was specified. Using last one (-1) as default (LActivation::Softmax)\n";
        }
        if (act_params.size() > 1)
            msg("Only one axis is supported (" + std::to_string(act_params.size()) + " were specified)", "LActivation::Softmax");
        const int last = (int)input->shape.size() - 1;
        if ((int)act_params[0] == -1) act_params[0] = (float)last;
        if ((int)act_params[0] == 0) msg("The axis of a softmax must not be the batch", "LActivation::Softmax");
        if ((int)act_params[0] < 0 || (int)act_params[0] > last)
            msg("The axis has to be a number from 0 to (number_of_dimensions - 1)", "LActivation::Softmax");
    }
    p->addchild(this);
    addparent(p);
}

void LActivation::forward() {
    if (act == "relu") tensorNN::ReLu(input, output);
    else if (act == "sigmoid") tensorNN::Sigmoid(input, output);
    else tensorNN::FullSoftmax(input, output, (int)act_params[0]);
}

// ---------------------------------------------------------------- pools
LPool::LPool(Layer *p, PoolDescriptor *D, const string &n, const string &prefix) : Layer(n, prefix), pd(D) {
    if (p->output->ndim != 4) msg("LPool only works over 4D tensors", "LPool::LPool");
    input = p->output;
    pd->build(input);
    output = pd->O;
    // src/layers/pool/layer_maxpool.cpp:46-51, layer_avgpool2D.cpp:43-48
    if (pd->pad[0] != pd->pad[1] || pd->pad[2] != pd->pad[3]) {
        string text = "In layer " + name + ": Padding asymmetry detected (top=" + std::to_string(pd->pad[0]) +
                      ", bottom=" + std::to_string(pd->pad[1]) + ", left=" + std::to_string(pd->pad[2]) +
                      ", right=" + std::to_string(pd->pad[3]) + "). The padding asymmetry is not allowed in a " +
                      (prefix == "maxpool2d" ? "MaxPool" : "AveragePool") +
                      " layer, we suggest you to use an explicit padding layer before this layer to fix the asymmetry.";
        vector<int> asym = pd->pad;
        delete pd;  // the output tensor stays with the Layer base, whose destructor releases it
        pd = nullptr;
        throw AsymmetricPaddingException(text, asym);
    }
    p->addchild(this);
    addparent(p);
}

LPool::~LPool() { delete pd; }

void LPool::resize(int batch) {
    pd->I = input;
    pd->resize(batch);
}

void LMaxPool::make_indices() {
    delete pd->indX;
    delete pd->indY;
    pd->indX = Tensor::zeros(pd->O->getShape(), pd->O->device);
    pd->indY = Tensor::zeros(pd->O->getShape(), pd->O->device);
}

LMaxPool::LMaxPool(Layer *p, const vector<int> &pool_size, const vector<int> &strides, const string &padding, string n)
    : LPool(p, new PoolDescriptor(pool_size, strides, padding, 0), n, "maxpool2d") {
    make_indices();
}

LMaxPool::LMaxPool(Layer *p, const vector<int> &pool_size, const vector<int> &strides, const vector<int> &padding, string n)
    : LPool(p, new PoolDescriptor(pool_size, strides, padding, 0), n, "maxpool2d") {
    make_indices();
}

void LMaxPool::forward() { tensorNN::MPool2D(pd); }

void LMaxPool::toGPU(int device) {
    Layer::toGPU(device);
    pd->indX->toGPU(device);
    pd->indY->toGPU(device);
}

void LMaxPool::resize(int batch) {
    LPool::resize(batch);
    make_indices();  // the index tensors are re-created with the output (src/layers/pool/layer_maxpool.cpp:50-60)
}

LAveragePool::LAveragePool(Layer *p, const vector<int> &pool_size, const vector<int> &strides, const string &padding, string n)
    : LPool(p, new PoolDescriptor(pool_size, strides, padding, 0), n, "avgpool") {}

LAveragePool::LAveragePool(Layer *p, const vector<int> &pool_size, const vector<int> &strides, const vector<int> &padding, string n)
    : LPool(p, new PoolDescriptor(pool_size, strides, padding, 0), n, "avgpool") {}

void LAveragePool::forward() { tensorNN::AvgPool2D(pd); }

// ---------------------------------------------------------------- LResize
LResize::LResize(Layer *p, vector<int> ns, string n) : Layer(n, "resize"), new_shape(ns) {
    input = p->output;
    output = new Tensor({input->shape[0], input->shape[1], new_shape[0], new_shape[1]}, DEV_CPU);
    p->addchild(this);
    addparent(p);
}

void LResize::forward() {
    // WrappingMode::Nearest = 2, TransformationMode::Asymmetric = 3 (include/eddl/utils.h:119-122)
    Tensor::scale(input, output, new_shape, 2, 0.0f, 3);
}

// ---------------------------------------------------------------- merges
LConcat::LConcat(vector<Layer *> ps, unsigned int ax, string n) : Layer(n, "concat") {
    if (ps.empty()) msg("Error: LConcat layer with empty list");
    if (ax == (unsigned)-1) ax = (ps[0]->output->ndim - 1) - 1;
    axis = ax;  // batch is not included
    if (ps.size() < 2) msg("Error: LConcat must receive at least two layers");
    const unsigned nd = ps[0]->output->ndim;
    if (axis + 1 >= nd) msg("The axis is out of range", "LConcat::LConcat");
    for (size_t i = 0; i + 1 < ps.size(); i++)
        if (nd != ps[i + 1]->output->ndim) msg("Error: LConcat layers with different tensor dims");
    for (size_t i = 0; i + 1 < ps.size(); i++)
        for (unsigned d = 0; d < nd; d++)
            if (d != axis + 1 && ps[i]->output->shape[d] != ps[i + 1]->output->shape[d])
                msg("Error: LConcat layers with different size in dim 1 (" + std::to_string(ps[i]->output->shape[d]) +
                    "!=" + std::to_string(ps[i + 1]->output->shape[d]) + ")");
    int t = 0;
    for (Layer *p : ps) t += p->output->shape[axis + 1];
    vector<int> ns = ps[0]->output->getShape();
    ns[axis + 1] = t;
    input = ps[0]->output;
    output = new Tensor(ns, DEV_CPU);
    for (Layer *p : ps) {
        p->addchild(this);
        addparent(p);
    }
}

void LConcat::forward() {
    vector<Tensor *> outs;
    for (Layer *p : parent) outs.push_back(p->output);
    Tensor::concat(outs, axis + 1, output);
}

LAdd::LAdd(vector<Layer *> ps, string n) : Layer(n, "add") {
    if (ps.empty()) msg("Error: LAdd layer with empty list");
    for (size_t i = 0; i + 1 < ps.size(); i++)
        if (ps[i]->output->shape != ps[i + 1]->output->shape) msg("Error: LAdd layers with different tensor shape");
    input = ps[0]->output;
    output = new Tensor(ps[0]->output->shape, DEV_CPU);
    for (Layer *p : ps) {
        p->addchild(this);
        addparent(p);
    }
}

void LAdd::forward() {
    output->fill_(0.0f);
    for (Layer *p : parent) Tensor::inc(p->output, output);
}

LSum::LSum(Layer *l1, Layer *l2, string n) : Layer(n, "sum") {
    if (l1->output->shape != l2->output->shape) msg("Error: LSum layers with different tensor shape", "LSum::LSum");
    input = l1->output;
    output = new Tensor(l1->output->shape, DEV_CPU);
    l1->addchild(this);
    l2->addchild(this);
    addparent(l1);
    addparent(l2);
}

void LSum::forward() { Tensor::add(1.0f, parent[0]->output, 1.0f, parent[1]->output, output, 0); }

// ---------------------------------------------------------------- LPad
LPad::LPad(Layer *p, vector<int> pads, float c, string n) : Layer(n, "pad"), constant(c) {
    if (pads.size() == 2) padding = {pads[0], pads[1], pads[0], pads[1]};
    else if (pads.size() == 4) padding = pads;
    else msg("The padding on each border must follow this format (top-bottom, left-right) or (top, right, bottom, left)", "LPad::LPad");
    input = p->output;
    if (input->ndim != 4) msg("This method requires two 4D tensors", "LPad::LPad");
    output = Tensor::full({input->shape[0], input->shape[1], input->shape[2] + (padding[0] + padding[2]),
                           input->shape[3] + (padding[1] + padding[3])},
                          constant, DEV_CPU);
    p->addchild(this);
    addparent(p);
}

void LPad::forward() { Tensor::pad(input, output, padding); }

// the border is written when the tensor is created; forward() copies the interior only
void LPad::resize(int batch) {
    output->resize(batch);
    output->fill_(constant);
}

void LPad::toGPU(int device) {
    Layer::toGPU(device);
    output->fill_(constant);
}

// ---------------------------------------------------------------- LReshape
LReshape::LReshape(Layer *p, vector<int> shape, string n) : Layer(n, "reshape"), ls(shape) {
    input = p->output;
    ls[0] = input->shape[0];
    const long tin = (long)input->size;
    long t = 1;
    int c = 0, ind = -1;
    for (size_t i = 0; i < ls.size(); i++) {
        if (ls[i] != -1) t *= ls[i];
        else if (c) msg("Ambiguous reshape, more than one -1", "Reshape");
        else {
            c = 1;
            ind = (int)i;
        }
    }
    if (c == 1) {
        if (t > tin || tin % t) msg("Incompatible shape", "Reshape");
        ls[ind] = (int)(tin / t);
    } else if (t != tin) {
        msg("Incompatible shape", "Reshape");
    }
    output = new Tensor(ls, input);  // shares the parent's storage
    p->addchild(this);
    addparent(p);
}

LReshape::~LReshape() {}  // the view does not own its storage (Tensor::release skips shared tensors)

void LReshape::resize(int batch) {
    // the parent has been resized already (layers are walked in forward order)
    ls[0] = batch;
    Tensor *old = output;
    output = new Tensor(ls, input);
    delete old;
    for (Layer *c : child) {  // children hold the tensor they read as `input`
        if (c->input == old) c->input = output;
    }
}

void LReshape::toGPU(int device) {
    dev = device;
    output->share(input);
}

// ---------------------------------------------------------------- LDense
LDense::LDense(Layer *p, int nd, bool ub, string n) : Layer(n, "dense"), ndim(nd), use_bias(ub) {
    input = p->output;
    vector<int> outshape(input->shape.begin(), input->shape.end() - 1);
    outshape.push_back(ndim);
    output = new Tensor(outshape, DEV_CPU);
    W = new Tensor(vector<int>{input->shape.back(), ndim}, DEV_CPU);
    params.push_back(W);
    if (use_bias) {
        bias = new Tensor(vector<int>{ndim}, DEV_CPU);
        params.push_back(bias);
    }
    p->addchild(this);
    addparent(p);
}

void LDense::forward() {
    const vector<int> inshape = input->shape, outshape = output->shape;
    input->reshape_({(int)(input->size / input->shape.back()), input->shape.back()});
    output->reshape_({(int)(output->size / output->shape.back()), output->shape.back()});
    Tensor::mult2D(input, 0, W, 0, output, 0);
    if (use_bias) Tensor::sum2D_rowwise(output, bias, output);
    input->reshape_(inshape);
    output->reshape_(outshape);
}

void LDense::initialize() {
    glorot_uniform(W);
    if (use_bias) bias->fill_(0.0f);
}

// ---------------------------------------------------------------- Net
namespace {
bool contains(const vector<Layer *> &v, Layer *l) {
    for (Layer *x : v)
        if (x == l) return true;
    return false;
}

// Net::walk (src/net/net.cpp:231-245)
void walk(Layer *l, const vector<Layer *> &lout, vector<Layer *> &seen) {
    if (contains(seen, l)) return;
    seen.push_back(l);
    if (contains(lout, l)) return;
    for (Layer *c : l->child) walk(c, lout, seen);
}

// Net::walk_back (src/net/net.cpp:248-258)
void walk_back(Layer *l, vector<Layer *> &seen) {
    if (contains(seen, l)) return;
    seen.push_back(l);
    for (Layer *p : l->parent) walk_back(p, seen);
}
}  // namespace

Net::Net(const vector<Layer *> &in, const vector<Layer *> &out) : lin(in), lout(out) {
    vector<Layer *> fwd, back;
    for (Layer *l : lin) walk(l, lout, fwd);
    for (Layer *l : lout) walk_back(l, back);
    vector<Layer *> all = fwd;
    for (Layer *l : back)
        if (!contains(all, l)) all.push_back(l);
    // Net::fts (src/net/net_build.cpp:34-70): always the first layer of the list whose parents are done
    vector<int> pending(all.size(), 0), taken(all.size(), 0);
    for (size_t i = 0; i < all.size(); i++)
        for (Layer *p : all[i]->parent)
            if (contains(all, p)) pending[i]++;
    for (size_t n = 0; n < all.size(); n++) {
        size_t j = 0;
        while (j < all.size() && !(pending[j] == 0 && !taken[j])) j++;
        if (j == all.size()) msg("error recurrent net", "Net.fts");
        taken[j] = 1;
        layers.push_back(all[j]);
        for (Layer *c : all[j]->child)
            for (size_t k = 0; k < all.size(); k++)
                if (all[k] == c) pending[k]--;
    }
    for (Layer *l : layers) l->net = this;
}

Net::~Net() {
    // an LInput's input and output are one tensor; LReshape outputs are views: both are handled by
    // the layers' destructors.  Layers are deleted children first so that views go before their base.
    for (size_t i = layers.size(); i-- > 0;) delete layers[i];
    delete cs;
}

void Net::build(CompServ *service, bool init_weights) {
    if (cs != nullptr) msg("the net has been built already", "Net::build");
    cs = service;
    int device = -1, count = 0;
    for (size_t i = 0; i < cs->local_gpus.size(); i++)
        if (cs->local_gpus[i]) {
            if (device < 0) device = (int)i;
            count++;
        }
    if (count == 0) msg("the computing service names no GPU", "Net::build");
    if (count > 1) msg("this backend runs a net on one GPU; the computing service names " + std::to_string(count), "Net::build");
    if (device >= gpu_devices()) msg("GPU " + std::to_string(device) + " is not present", "Net::build");
    gpu_init(device);
    dev = DEV_GPU + device;
    for (Layer *l : layers) l->toGPU(dev);
    // the parameters are drawn on the device, as the reference draws those of the device copy of a net
    if (init_weights)
        for (Layer *l : layers) l->initialize();
}

void Net::resize(int batch) {
    if (batch == batch_size) return;
    batch_size = batch;
    for (Layer *l : layers) l->resize(batch);
}

void Net::setmode(int m) {
    for (Layer *l : layers) l->setmode(m);
}

void Net::forward() {
    ProfileScope profile(profile_forward());
    if (plan.empty()) {
        for (Layer *l : layers) l->forward();
        return;
    }
    // the steps are queued in order on the device's stream; one wait at the end
    const bool was_synchronous = gpu_get_synchronous();
    gpu_set_synchronous(false);
    try {
        for (const FusedStep &s : plan) run_step(s);
    } catch (...) {
        gpu_set_synchronous(was_synchronous);
        throw;
    }
    gpu_set_synchronous(was_synchronous);
    if (was_synchronous) gpu_synchronize(dev - DEV_GPU);
}

bool Net::is_fused_away(const Layer *l) const {
    for (const Layer *x : fused_away)
        if (x == l) return true;
    return false;
}

// The chains follow one rule: a layer is taken into the step of the layer before it only when it is
// that layer's sole child and the layer before it is not an output of the net, so that nothing else
// reads the tensor that is no longer written.
void Net::fuse() {
    if (dev == DEV_CPU) msg("build the net with a computing service first", "Net::fuse");
    plan.clear();
    fused_away.clear();
    auto sole_child = [this](Layer *l) -> Layer * { return (l->child.size() == 1 && !contains(lout, l)) ? l->child[0] : nullptr; };
    vector<Layer *> done;      // layers whose output tensor the plan writes
    vector<Layer *> absorbed;  // layers computed by the step of an earlier layer
    for (Layer *l : layers) {
        if (contains(absorbed, l)) continue;
        FusedStep s;
        s.first = s.last = l;
        if (LPad *pad = dynamic_cast<LPad *>(l)) {
            Layer *c = sole_child(l);
            if (pad->constant == 0.0f && c != nullptr && dynamic_cast<LConv *>(c) != nullptr) {
                fused_away.push_back(l);  // the convolution reads the pad's parent with larger paddings
                continue;
            }
        }
        if (LResize *rs = dynamic_cast<LResize *>(l)) {
            // a nearest upsampling by whole factors read only by a 1x1, 2x2 or 3x3 convolution, directly or through a zero
            // pad that the convolution absorbs: folded into the convolution's gather (eddlhip_conv2d_fwd_upsampled)
            Layer *c = sole_child(l);
            if (LPad *pad = dynamic_cast<LPad *>(c))
                if (pad->constant == 0.0f) c = sole_child(pad);
            LConv *cv = dynamic_cast<LConv *>(c);
            const Tensor *in = rs->parent[0]->output;
            if (cv != nullptr && in->ndim == 4 && rs->new_shape[0] % in->shape[2] == 0 && rs->new_shape[1] % in->shape[3] == 0 &&
                cv->cd->kernel_size[0] == cv->cd->kernel_size[1] && cv->cd->kernel_size[0] >= 1 && cv->cd->kernel_size[0] <= 3) {
                fused_away.push_back(l);
                continue;
            }
        }
        if (LConcat *cat = dynamic_cast<LConcat *>(l)) {
            // a channel Concat of two equal-shaped 4-D tensors read only by a 1x1, 2x2 or 3x3 convolution: that
            // convolution takes the two halves of its channels from the two tensors (eddlhip_conv2d_fwd_concat)
            LConv *cv = dynamic_cast<LConv *>(sole_child(l));
            if (cv != nullptr && cat->axis == 0 && cat->parent.size() == 2 && cat->parent[0] != cat->parent[1] &&
                cat->output->ndim == 4 && cat->parent[0]->output->shape == cat->parent[1]->output->shape &&
                cv->cd->kernel_size[0] == cv->cd->kernel_size[1] && cv->cd->kernel_size[0] >= 1 && cv->cd->kernel_size[0] <= 3) {
                fused_away.push_back(l);
                continue;
            }
        }
        if (LConv *conv = dynamic_cast<LConv *>(l)) {
            // the steps call the library directly, past tensorNN::Conv2D and its check (src/tensor/nn/tensor_conv.cpp:48-51)
            if (conv->cd->dilation_rate[0] != 1 || conv->cd->dilation_rate[1] != 1)
                msg("Dilated convolutions are only available with CuDNN", "Net::fuse");
            s.chain = true;
            s.src = l->parent[0];
            s.pad_top = conv->cd->padrt;
            s.pad_left = conv->cd->padcl;
            if (LPad *pad = dynamic_cast<LPad *>(s.src)) {
                if (is_fused_away(pad)) {
                    s.pad_top += pad->padding[0];   // (top, right, bottom, left)
                    s.pad_left += pad->padding[3];
                    s.src = pad->parent[0];
                }
            }
            if (LResize *rs = dynamic_cast<LResize *>(s.src)) {
                if (is_fused_away(rs)) {
                    s.src = rs->parent[0];
                    s.up_h = rs->new_shape[0] / s.src->output->shape[2];
                    s.up_w = rs->new_shape[1] / s.src->output->shape[3];
                }
            }
            if (LConcat *cat = dynamic_cast<LConcat *>(s.src)) {
                if (is_fused_away(cat)) {
                    s.src = cat->parent[0];
                    s.src2 = cat->parent[1];
                }
            }
            Layer *c = sole_child(s.last);
            if (LBatchNorm *bn = dynamic_cast<LBatchNorm *>(c)) {
                s.bn = bn;
                s.last = bn;
                c = sole_child(s.last);
            }
            if (LSum *sum = dynamic_cast<LSum *>(c)) {
                Layer *other = sum->parent[0] == s.last ? sum->parent[1] : sum->parent[0];
                if (other != s.last && contains(done, other)) {
                    s.res = other;
                    s.last = sum;
                    c = sole_child(s.last);
                }
            } else if (LAdd *add = dynamic_cast<LAdd *>(c)) {
                // an LAdd of two layers computes (0 + a) + b, which differs from a + b only in the sign of a
                // zero result; a ReLU behind it maps both to +0, so the pair is taken only together
                if (add->parent.size() == 2) {
                    Layer *other = add->parent[0] == s.last ? add->parent[1] : add->parent[0];
                    LActivation *nxt = dynamic_cast<LActivation *>(sole_child(add));
                    if (other != s.last && contains(done, other) && nxt != nullptr && nxt->act == "relu") {
                        s.res = other;
                        s.last = add;
                        c = nxt;
                    }
                }
            }
            if (LActivation *a = dynamic_cast<LActivation *>(c)) {
                if (a->act == "relu") {
                    s.relu = true;
                    s.last = a;
                }
            }
            for (Layer *m = l; m != s.last; m = m->child[0]) {
                fused_away.push_back(m);
                absorbed.push_back(m->child[0]);
            }
            // a 2x2, stride-2, unpadded LMaxPool of the chain's output joins the call (eddlhip_conv2d_fwd_maxpool: a
            // convolution in a Winograd form pools in its epilogue); the unpooled tensor is written only if read elsewhere
            if (conv->cd->r % 2 == 0 && conv->cd->c % 2 == 0) {
                for (Layer *c2 : s.last->child) {
                    LMaxPool *mp = dynamic_cast<LMaxPool *>(c2);
                    if (mp == nullptr || mp->parent.size() != 1) continue;
                    const PoolDescriptor *pd = mp->pd;
                    if (pd->ksize != vector<int>{2, 2} || pd->stride != vector<int>{2, 2} || pd->pad != vector<int>{0, 0, 0, 0}) continue;
                    s.pool = mp;
                    s.keep = s.last->child.size() > 1 || contains(lout, s.last);
                    absorbed.push_back(mp);
                    done.push_back(mp);
                    if (!s.keep) fused_away.push_back(s.last);
                    break;
                }
            }
        } else if (dynamic_cast<LDense *>(l) != nullptr) {
            s.chain = true;
            LActivation *a = dynamic_cast<LActivation *>(sole_child(l));
            if (a != nullptr && a->act == "relu") {
                s.relu = true;
                s.last = a;
                fused_away.push_back(l);
                absorbed.push_back(a);
            }
        }
        done.push_back(s.last);
        plan.push_back(s);
    }
    for (Layer *o : lout)
        if (is_fused_away(o)) msg("output layer " + o->name + " was fused away", "Net::fuse");
    for (Layer *l : layers)
        if (LConv *conv = dynamic_cast<LConv *>(l))
            gpu_check(eddlhip_conv2d_cache_filters(dev - DEV_GPU, conv->cd->K->ptr, conv->cd->nk, conv->cd->kz, conv->cd->kr, conv->cd->kc),
                      "Net::fuse");
}

void Net::run_step(const FusedStep &s) {
    if (!s.chain) {
        s.first->forward();
        return;
    }
    const int device = dev - DEV_GPU;
    if (LConv *conv = dynamic_cast<LConv *>(s.first)) {
        const ConvolDescriptor *D = conv->cd;
        const Tensor *I = s.src->output;
        Tensor *O = s.last->output;
        const LBatchNorm *bn = s.bn;
        // the step computes the inference form; the layer walk would raise in gpu_batchnorm_forward
        if (bn != nullptr && bn->mode == TRMODE)
            msg("training-mode batch normalisation is outside this forward/inference backend", "Net::forward (fused convolution)");
        const float *bias = D->use_bias ? D->bias->ptr : nullptr;
        const float *g = bn && bn->affine ? bn->bn_g->ptr : nullptr, *b = bn && bn->affine ? bn->bn_b->ptr : nullptr;
        const float *mean = bn ? bn->mean->ptr : nullptr, *var = bn ? bn->variance->ptr : nullptr;
        const float eps = bn ? bn->epsilon : 0.0f;
        const float *res = s.res ? s.res->output->ptr : nullptr;
        if (s.pool != nullptr) {
            const int c_in = s.src2 != nullptr ? 2 * I->shape[1] : I->shape[1];
            gpu_check(eddlhip_conv2d_fwd_maxpool(device, I->ptr, s.src2 != nullptr ? s.src2->output->ptr : nullptr, s.up_h, s.up_w, D->K->ptr, bias,
                                                 O->ptr, I->shape[0], c_in, I->shape[2], I->shape[3], D->nk, D->kr, D->kc, D->sr, D->sc,
                                                 s.pad_top, s.pad_left, D->r, D->c, g, b, mean, var, eps, res, s.relu ? 1 : 0,
                                                 s.pool->output->ptr, s.pool->pd->indX->ptr, s.pool->pd->indY->ptr, s.keep ? 1 : 0),
                      "Net::forward (fused convolution and max-pool)");
            return;
        }
        if (s.up_h != 1 || s.up_w != 1)
            gpu_check(eddlhip_conv2d_fwd_upsampled(device, I->ptr, s.up_h, s.up_w, D->K->ptr, bias, O->ptr, I->shape[0], I->shape[1],
                                                   I->shape[2], I->shape[3], D->nk, D->kr, D->kc, D->sr, D->sc, s.pad_top, s.pad_left,
                                                   D->r, D->c, g, b, mean, var, eps, res, s.relu ? 1 : 0),
                      "Net::forward (fused convolution over an upsampled tensor)");
        else if (s.src2 != nullptr)
            gpu_check(eddlhip_conv2d_fwd_concat(device, I->ptr, s.src2->output->ptr, D->K->ptr, bias, O->ptr, I->shape[0], 2 * I->shape[1],
                                                I->shape[2], I->shape[3], D->nk, D->kr, D->kc, D->sr, D->sc, s.pad_top, s.pad_left, D->r,
                                                D->c, g, b, mean, var, eps, res, s.relu ? 1 : 0),
                      "Net::forward (fused convolution over two tensors)");
        else
            gpu_check(eddlhip_conv2d_fwd(device, I->ptr, D->K->ptr, bias, O->ptr, I->shape[0], I->shape[1], I->shape[2], I->shape[3], D->nk,
                                         D->kr, D->kc, D->sr, D->sc, s.pad_top, s.pad_left, D->r, D->c, g, b, mean, var, eps, res,
                                         s.relu ? 1 : 0),
                      "Net::forward (fused convolution)");
        return;
    }
    LDense *dense = static_cast<LDense *>(s.first);
    const Tensor *A = dense->input;
    const int k = A->shape.back(), n = dense->ndim;
    gpu_check(eddlhip_dense_fwd(device, A->ptr, dense->W->ptr, dense->use_bias ? dense->bias->ptr : nullptr, s.last->output->ptr,
                                (int)(A->size / k), k, n, s.relu ? 1 : 0),
              "Net::forward (fused dense)");
}

void Net::forward(const vector<Tensor *> &in) {
    if (dev == DEV_CPU) msg("build the net with a computing service first", "Net.forward(vtensor)");
    if (!in.empty()) {
        if (in.size() != lin.size()) msg("size missmatch in list of tensors", "Net.forward(vtensor)");
        if (batch_size != in[0]->shape[0]) resize(in[0]->shape[0]);
        for (size_t i = 0; i < in.size(); i++) Tensor::copy(in[i], lin[i]->output);
    }
    forward();
}

vector<Tensor *> Net::predict(const vector<Tensor *> &in) {
    setmode(TSMODE);
    forward(in);
    vector<Tensor *> out;
    for (Layer *l : lout) {
        Tensor *t = new Tensor(l->output->getShape(), DEV_CPU);
        Tensor::copy(l->output, t);
        out.push_back(t);
    }
    return out;
}

// "bin" files: for every layer in `layers` order, for every parameter in the layer's order,
// int32 ndim | int32 shape[ndim] | float32 data (src/net/net.cpp:411-449, src/layers/layer.cpp:215-227,
// src/tensor/tensor_serialization.cpp:70-110,252-261)
void Net::save(const string &filename, const string &format) {
    if (format != "bin") msg("Format not implemented: *.'" + format + "'", "Tensor::save");
    std::ofstream ofs(filename, std::ios::out | std::ios::binary);
    for (Layer *l : layers)
        for (Tensor *p : l->params) {
            Tensor host(p->getShape(), DEV_CPU);
            Tensor::copy(p, &host);
            int nd = (int)host.ndim;
            ofs.write(reinterpret_cast<const char *>(&nd), sizeof(int));
            ofs.write(reinterpret_cast<const char *>(host.shape.data()), host.shape.size() * sizeof(int));
            ofs.write(reinterpret_cast<const char *>(host.ptr), host.size * sizeof(float));
        }
}

void Net::load(const string &filename, const string &format) {
    if (format != "bin") msg("Format not implemented: *.'" + format + "'", "Tensor::load");
    std::ifstream ifs(filename, std::ios::in | std::ios::binary);
    if (!ifs.good()) throw std::runtime_error(string("File not found. Check the file name and try again (Net::load)"));
    for (Layer *l : layers)
        for (Tensor *p : l->params) {
            int nd = 0;
            ifs.read(reinterpret_cast<char *>(&nd), sizeof(int));
            if (!ifs.good() || nd < 0 || nd > 8) msg("the file ends early or is not in the bin format (layer " + l->name + ")", "Net::load");
            vector<int> shape(nd);
            ifs.read(reinterpret_cast<char *>(shape.data()), nd * sizeof(int));
            // (a record is trusted only as far as it fits the parameter it is for: nothing is allocated from a size the file names)
            unsigned long long count = ifs.good() ? 1 : 0;
            for (int d : shape) count = (d > 0 && count <= p->size) ? count * (unsigned long long)d : 0;
            if (count != p->size)
                msg("a record of the file does not hold the " + std::to_string(p->size) + " values of a parameter of layer " + l->name, "Net::load");
            Tensor host(shape, DEV_CPU);
            ifs.read(reinterpret_cast<char *>(host.ptr), host.size * sizeof(float));
            if (!ifs.good()) msg("the file ends inside a parameter of layer " + l->name, "Net::load");
            Tensor::copy(&host, p);  // any shape of the same size, as the reference's copy accepts
        }
}

vector<vector<Tensor *>> Net::get_parameters(bool) {
    vector<vector<Tensor *>> all;
    for (Layer *l : layers) {
        vector<Tensor *> ps;
        for (Tensor *p : l->params) {
            Tensor *host = new Tensor(p->getShape(), DEV_CPU);
            Tensor::copy(p, host);
            ps.push_back(host);
        }
        all.push_back(ps);
    }
    return all;
}

void Net::set_parameters(const vector<vector<Tensor *>> &new_params) {
    if (new_params.size() != layers.size())
        msg("AssertionError: The number of layers in params does not match the number of layers in this network (" +
                std::to_string(new_params.size()) + "!=" + std::to_string(layers.size()) + ")",
            "Net::set_parameters");
    for (size_t i = 0; i < layers.size(); i++)
        if (new_params[i].size() != layers[i]->params.size())
            msg("AssertionError: The number of parameters in layer '" + std::to_string(i) + "'(" + layers[i]->name +
                    ") does not match the number of parameters in the given vector<Tensor*>. (" +
                    std::to_string(layers[i]->params.size()) + "!=" + std::to_string(new_params[i].size()) + ")",
                "Net::set_parameters");
    for (size_t i = 0; i < layers.size(); i++)
        for (size_t j = 0; j < layers[i]->params.size(); j++) Tensor::copy(new_params[i][j], layers[i]->params[j]);
}

Layer *Net::getLayer(const string &lname) {
    for (Layer *l : layers)
        if (l->name == lname) return l;
    msg("layer " + lname + " not found", "Net::getLayer");
    return nullptr;
}

string Net::summary(bool print_stdout) {
    std::stringstream ss;
    ss << "-------------------------------------------------------------------------------\n" << name << "\n";
    ss << "-------------------------------------------------------------------------------\n";
    size_t maxl = 0;
    for (Layer *l : layers) maxl = std::max(maxl, l->name.size());
    long total = 0;
    for (Layer *l : layers) {
        long np = 0;
        for (Tensor *p : l->params) np += (long)p->size;
        total += np;
        auto shp = [](const vector<int> &s) {
            string r = "(";
            for (size_t i = 1; i < s.size(); i++) r += (i > 1 ? ", " : "") + std::to_string(s[i]);
            return r + ")";
        };
        ss << std::setw((int)maxl) << std::left << l->name << "|  " << std::setw(20) << shp(l->input->shape) << "=>   " << std::setw(20)
           << shp(l->output->shape) << std::setw(12) << np << "\n";
    }
    ss << "-------------------------------------------------------------------------------\n";
    ss << "Total params: " << total << "\n";
    if (print_stdout) std::cout << ss.str();
    return ss.str();
}

// ---------------------------------------------------------------- eddl:: API
namespace eddl {

model Model(vlayer in, vlayer out) { return new Net(in, out); }
void setName(model m, string name) { m->name = name; }

compserv CS_HIP(const vector<int> &g, const string &mem) {
    CompServ *cs = new CompServ();
    cs->local_gpus = g;
    cs->mem = mem;
    return cs;
}
compserv CS_GPU(const vector<int> &g, const string &mem) { return CS_HIP(g, mem); }

void build(model net, compserv cs, bool init_weights) { net->build(cs, init_weights); }
void fuse(model net) { net->fuse(); }
void show_profile() { __show_profile(); }
void reset_profile() { __reset_profile(); }
void set_mode(model net, int mode) { net->setmode(mode); }
void summary(model m) { m->summary(true); }
void load(model m, const string &fname, const string &format) { m->load(fname, format); }
void save(model m, const string &fname, const string &format) { m->save(fname, format); }

vlayer forward(model m, vtensor in) {
    m->forward(in);
    return m->lout;
}

vtensor predict(model m, const vtensor &in) { return m->predict(in); }

Tensor *getOutput(layer l1) {
    if (l1->net != nullptr && l1->net->is_fused_away(l1))
        msg("layer " + l1->name + " is computed inside a fused step of the plan; its output is not kept", "getOutput");
    Tensor *t = new Tensor(l1->output->getShape(), DEV_CPU);
    Tensor::copy(l1->output, t);
    return t;
}

vector<vtensor> get_parameters(model net, bool deepcopy) { return net->get_parameters(deepcopy); }
void set_parameters(model net, const vector<vtensor> &params) { net->set_parameters(params); }
layer getLayer(model net, const string &name) { return net->getLayer(name); }
vlayer getOut(model net) { return net->lout; }
vtensor getParams(layer l1) {
    vtensor out;
    for (Tensor *p : l1->params) {
        Tensor *host = new Tensor(p->getShape(), DEV_CPU);
        Tensor::copy(p, host);
        out.push_back(host);
    }
    return out;
}

layer Input(const vector<int> &shape, string name) {
    vector<int> s(shape);
    s.insert(s.begin(), 1);  // batch 1 until a forward says otherwise (src/apis/eddl.cpp:604-608)
    return new LInput(new Tensor(s, DEV_CPU), name);
}

layer Conv2D(layer parent, int filters, const vector<int> &kernel_size, const vector<int> &strides, string padding, bool use_bias,
             int groups, const vector<int> &dilation_rate, string name) {
    return new LConv(parent, filters, kernel_size, strides, padding, {}, groups, dilation_rate, use_bias, name);
}

layer Dense(layer parent, int ndim, bool use_bias, string name) { return new LDense(parent, ndim, use_bias, name); }

layer Activation(layer parent, string activation, vector<float> params, string name) {
    return new LActivation(parent, activation, params, name);
}
layer ReLu(layer parent, string name) { return new LActivation(parent, "relu", {}, name); }
layer Sigmoid(layer parent, string name) { return new LActivation(parent, "sigmoid", {}, name); }
layer Softmax(layer parent, int axis, string name) { return new LActivation(parent, "softmax", {(float)axis}, name); }

layer BatchNormalization(layer parent, float momentum, float epsilon, bool affine, string name) {
    return new LBatchNorm(parent, momentum, epsilon, affine, name);
}
layer BatchNormalization(layer parent, bool affine, float momentum, float epsilon, string name) {
    return new LBatchNorm(parent, momentum, epsilon, affine, name);
}

layer MaxPool2D(layer parent, vector<int> pool_size, vector<int> strides, string padding, string name) {
    return new LMaxPool(parent, pool_size, strides, padding, name);
}
layer AveragePool2D(layer parent, vector<int> pool_size, vector<int> strides, string padding, string name) {
    return new LAveragePool(parent, pool_size, strides, padding, name);
}
layer AvgPool2D(layer parent, vector<int> pool_size, vector<int> strides, string padding, string name) {
    return AveragePool2D(parent, pool_size, strides, padding, name);
}
layer GlobalAveragePool2D(layer parent, string name) {
    if (parent->output->ndim != 4) msg("GlobalAveragePool only works over 4D tensors", "GlobalAveragePool2D");
    if (name.empty()) name = "GlobalAveragePool2D";
    return AveragePool2D(parent, {parent->output->shape[2], parent->output->shape[3]}, {1, 1}, "none", name);
}

layer UpSampling2D(layer parent, const vector<int> &size, string interpolation, string name) {
    if (interpolation != "nearest")
        std::cerr << "Warning: In UpSampling2D the interpolation type \"" << interpolation
                  << "\" is not valid. Only \"nearest\" is available.\n";
    const vector<int> ps = parent->output->getShape();
    if (ps.size() != 4) msg("The number of dimensions of the input tensor must be 4", "EDDL::UpSampling2D");
    if (size.size() != 2) msg("The number of dimensions of the \"size\" parameter must be 2", "EDDL::UpSampling2D");
    vector<int> target;
    for (int i : {2, 3}) {
        if (size[i - 2] < 1) msg("The scale factors in \"size\" parameter must be greater or equal to 1", "EDDL::UpSampling2D");
        target.push_back(ps[i] * size[i - 2]);
    }
    return new LResize(parent, target, name);
}

layer Concat(const vector<layer> &layers, unsigned int axis, string name) { return new LConcat(layers, axis, name); }
layer Add(const vector<layer> &layers, string name) { return new LAdd(layers, name); }
layer Add(layer l1, layer l2) { return new LSum(l1, l2, ""); }
layer Pad(layer parent, vector<int> padding, float constant, string name) { return new LPad(parent, padding, constant, name); }

layer Reshape(layer parent, const vector<int> &shape, string name) {
    vector<int> s(shape);
    s.insert(s.begin(), 1);
    return new LReshape(parent, s, name);
}
layer Flatten(layer parent, string name) { return Reshape(parent, {-1}, name); }

}  // namespace eddl
}  // namespace eddl_hip
