// Module / Sequential / the layers of the benchmark's MLP and CNN, and the optimizers that finish a training
// step. API as in the reference's include/origin/nn/** and include/origin/optim/**; these are callers of the hot
// path (host glue), not kernels.
#pragma once
#include <functional>
#include <memory>
#include <string>
#include <unordered_map>
#include <vector>

#include <any>

#include "functional.h"
#include "io.h"

namespace origin
{
class Module
{
public:
    Module() : training_(true) {}
    virtual ~Module() = default;
    virtual Tensor forward(const Tensor &input) = 0;
    Tensor operator()(const Tensor &input) { return forward(input); }
    virtual std::vector<Parameter *> parameters();
    void register_parameter(const std::string &name, Parameter &param);
    void register_module(const std::string &name, std::unique_ptr<Module> module);
    // name -> tensor of every registered parameter, children prefixed "child." (src/nn/module.cpp:120-207)
    using StateDict = std::unordered_map<std::string, Tensor>;
    virtual StateDict state_dict() const;
    virtual void load_state_dict(const StateDict &state_dict, bool strict = true);
    void load(const std::string &filepath, bool strict = true);
    std::unordered_map<std::string, Parameter *> named_parameters(const std::string &prefix = "");
    std::unordered_map<std::string, const Parameter *> named_parameters(const std::string &prefix) const;
    void train(bool mode = true);
    void eval() { train(false); }
    bool is_training() const { return training_; }
    virtual void to(Device device);
    void zero_grad();

protected:
    std::vector<std::pair<std::string, Parameter *>> parameters_;         // registration order
    std::vector<std::pair<std::string, std::unique_ptr<Module>>> modules_;
    bool training_;
};

using Layer = Module;  // the reference's layers derive from an empty Layer : Module

class Sequential : public Module
{
public:
    void add(std::unique_ptr<Module> module) { layers_.push_back(std::move(module)); }
    Tensor forward(const Tensor &input) override;
    std::vector<Parameter *> parameters() override;
    void to(Device device) override;
    Module &operator[](size_t index) { return *layers_.at(index); }
    const Module &operator[](size_t index) const { return *layers_.at(index); }
    size_t size() const { return layers_.size(); }

private:
    std::vector<std::unique_ptr<Module>> layers_;
};

namespace nn
{
// weight [in, out] = randn * sqrt(1/in), bias zeros [1, out] (src/nn/layers/linear.cpp:39-62)
class Linear : public Module
{
public:
    Linear(int in_features, int out_features, bool bias = true);
    Tensor forward(const Tensor &input) override;
    // relu(forward(input)); Sequential calls it for a Linear that a ReLU follows, and on the device the two run as one
    Tensor forward_relu(const Tensor &input);
    Parameter *weight() { return &weight_; }
    Parameter *bias() { return use_bias_ ? &bias_ : nullptr; }
    void reset_parameters();

private:
    int in_features_, out_features_;
    bool use_bias_;
    Parameter weight_, bias_;
};

// weight [OC, C, KH, KW] = randn * sqrt(2/fan_in), bias zeros [OC] (src/nn/layers/conv2d.cpp:78-103)
class Conv2d : public Module
{
public:
    Conv2d(int in_channels, int out_channels, std::pair<int, int> kernel_size, std::pair<int, int> stride = {1, 1},
           std::pair<int, int> pad = {0, 0}, bool bias = true);
    Conv2d(int in_channels, int out_channels, int kernel_size, int stride = 1, int pad = 0, bool bias = true);
    Tensor forward(const Tensor &input) override;
    Tensor forward_relu(const Tensor &input);  // relu(forward(input)), as Linear::forward_relu
    // max_pool2d(relu(forward(input)), ...) as one operator
    Tensor forward_relu_pool(const Tensor &input, std::pair<int, int> pool_kernel, std::pair<int, int> pool_stride,
                             std::pair<int, int> pool_pad);
    Parameter *weight() { return &weight_; }
    Parameter *bias() { return use_bias_ ? &bias_ : nullptr; }

private:
    int in_channels_, out_channels_;
    std::pair<int, int> kernel_, stride_, pad_;
    bool use_bias_;
    Parameter weight_, bias_;
};

class MaxPool2d : public Module
{
public:
    MaxPool2d(std::pair<int, int> kernel_size, std::pair<int, int> stride = {0, 0}, std::pair<int, int> pad = {0, 0});
    MaxPool2d(int kernel_size, int stride = 0, int pad = 0);
    Tensor forward(const Tensor &input) override { return functional::max_pool2d(input, kernel_, stride_, pad_); }
    std::pair<int, int> kernel_size() const { return kernel_; }
    std::pair<int, int> stride() const { return stride_; }
    std::pair<int, int> pad() const { return pad_; }

private:
    std::pair<int, int> kernel_, stride_, pad_;
};

class ReLU : public Module
{
public:
    Tensor forward(const Tensor &input) override { return functional::relu(input); }
};

class Flatten : public Module
{
public:
    explicit Flatten(int start_dim = 1, int end_dim = -1) : start_(start_dim), end_(end_dim) {}
    Tensor forward(const Tensor &input) override { return functional::flatten(input, start_, end_); }

private:
    int start_, end_;
};

// gamma ones, beta zeros, running mean zeros, running variance ones (src/nn/layers/batch_norm2d.cpp:12-35). In
// training mode each forward normalises with the batch statistics and then folds them into the running ones as
// running = momentum * running + (1 - momentum) * batch (batch_norm2d.cpp:62-86: this order, not the usual one);
// in evaluation mode the running statistics are used. The update is one device launch per statistic here; the
// reference copies four vectors to the host and two back. Only gamma ("weight") and beta ("bias") are registered
// parameters, as in the reference, but to(device) also moves the running statistics.
class BatchNormBase : public Module
{
public:
    Tensor forward(const Tensor &input) override;
    // relu(forward(input)) as one operator on a float32 device tensor: the normalised tensor is never stored, and in
    // backward the ReLU's mask is formed again inside the normalisation's own kernels (same values either way)
    Tensor forward_relu(const Tensor &input);
    Parameter *weight() { return &gamma_; }
    Parameter *bias() { return &beta_; }
    const Tensor &running_mean() const { return running_mean_; }
    const Tensor &running_var() const { return running_var_; }
    void reset_parameters();
    void to(Device device) override;
    using Module::to;

protected:
    BatchNormBase(const char *name, int num_dims, int num_features, float eps, float momentum);
    Tensor run(const Tensor &input, bool relu);
    const char *name_;
    int num_dims_, num_features_;
    float eps_, momentum_;
    Parameter gamma_, beta_;
    Tensor running_mean_, running_var_;
};

class BatchNorm1d : public BatchNormBase  // input [N, C] (src/nn/layers/batch_norm1d.cpp)
{
public:
    explicit BatchNorm1d(int num_features, float eps = 1e-5f, float momentum = 0.1f)
        : BatchNormBase("BatchNorm1d", 2, num_features, eps, momentum)
    {}
};

class BatchNorm2d : public BatchNormBase  // input [N, C, H, W] (src/nn/layers/batch_norm2d.cpp)
{
public:
    explicit BatchNorm2d(int num_features, float eps = 1e-5f, float momentum = 0.1f)
        : BatchNormBase("BatchNorm2d", 4, num_features, eps, momentum)
    {}
};

// MLP({784, 1000, 10}, relu): Linear layers with the activation between them, none after the last
// (src/nn/models/mlp.cpp:11-61)
class MLP : public Module
{
public:
    MLP(const std::vector<int> &sizes, std::function<Tensor(const Tensor &)> activation = nullptr);
    Tensor forward(const Tensor &input) override;
    Linear &layer(size_t i) { return *layers_.at(i); }
    size_t num_layers() const { return layers_.size(); }

private:
    std::vector<Linear *> layers_;
    std::function<Tensor(const Tensor &)> activation_;
    bool default_relu_ = false;  // no activation was given: the ReLU between the layers rides in their epilogues
};
}  // namespace nn

// ------------------------------------------------------------------------------------------ optimizers
class Optimizer
{
public:
    explicit Optimizer(Module &target);
    virtual ~Optimizer() = default;
    void step();       // filter params with a gradient -> hooks -> step_one each (src/optim/optimizer.cpp:19-53)
    void zero_grad();
    void register_hook(std::function<void(std::vector<Parameter *> &)> hook) { hooks_.push_back(std::move(hook)); }
    // settings as float / bool values, buffers as StateDict values keyed "<kind>_<parameter name>"
    // (src/optim/adam.cpp:116-284, src/optim/sgd.cpp:77-157)
    virtual std::unordered_map<std::string, std::any> state_dict() const = 0;
    virtual void load_state_dict(const std::unordered_map<std::string, std::any> &state_dict) = 0;
    // Call before every replay of a graph that recorded step(): brings the host-side state the recorded kernels
    // depend on (Adam's step counts and bias-correction factors) forward by one step. While a graph is being
    // captured, step() writes parameters and buffers in place, so that replays find them at the recorded addresses;
    // at least one ordinary step must have run before (the buffers must exist).
    virtual void prepare_replay() {}

protected:
    virtual void step_one(Parameter &param) = 0;
    // all parameters that have a gradient, after the hooks: one by one unless the optimizer knows better
    virtual void step_all(std::vector<Parameter *> &params)
    {
        for (auto *p : params)
            step_one(*p);
    }
    // true when step_all will update this list in one launch that can apply a WeightDecay hook on its way: step() then
    // hands the hook's rate over in hook_decay_ instead of running the hook as a launch of its own (same floats)
    virtual bool step_all_takes_decay(const std::vector<Parameter *> &) const { return false; }
    float hook_decay_ = 0.0f;
    Module *target_;
    std::vector<Parameter *> parameters_;
    std::vector<std::function<void(std::vector<Parameter *> &)>> hooks_;
};

class SGD : public Optimizer  // src/optim/sgd.cpp:18-75
{
public:
    SGD(Module &target, float lr, float momentum = 0.0f, float weight_decay = 0.0f, bool nesterov = false);
    std::unordered_map<std::string, std::any> state_dict() const override;
    void load_state_dict(const std::unordered_map<std::string, std::any> &state_dict) override;

protected:
    void step_one(Parameter &param) override;
    void step_all(std::vector<Parameter *> &params) override;
    bool step_all_takes_decay(const std::vector<Parameter *> &params) const override;

private:
    float lr_, momentum_, weight_decay_;
    bool nesterov_;
    std::unordered_map<Parameter *, Tensor> momentum_buffers_;
};

class Adam : public Optimizer  // src/optim/adam.cpp:19-114
{
public:
    Adam(Module &target, float lr = 0.001f, float beta1 = 0.9f, float beta2 = 0.999f, float eps = 1e-8f);
    std::unordered_map<std::string, std::any> state_dict() const override;
    void load_state_dict(const std::unordered_map<std::string, std::any> &state_dict) override;

protected:
    void step_one(Parameter &param) override;
    void step_all(std::vector<Parameter *> &params) override;
    bool step_all_takes_decay(const std::vector<Parameter *> &params) const override;

private:
    float lr_, beta1_, beta2_, eps_;
    std::unordered_map<Parameter *, Tensor> m_buffers_, v_buffers_;
    std::unordered_map<Parameter *, int> step_counts_;
    Tensor replay_scales_;                      // [parameters, 2] on the device: 1/(1-b1^t), 1/(1-b2^t) per parameter
    std::vector<Parameter *> replay_params_;    // the parameters the recorded step updates

public:
    void prepare_replay() override;
};

// what WeightDecay::hook() wraps: a named type, so that Optimizer::step can recognise the hook and its rate
struct WeightDecayHook
{
    float rate;
    void operator()(std::vector<Parameter *> &params) const;
};

class WeightDecay  // include/origin/optim/hooks.h:37-66: grad += rate * param, for every parameter
{
public:
    explicit WeightDecay(float rate = 1e-4f) : rate_(rate) {}
    std::function<void(std::vector<Parameter *> &)> hook() const;

private:
    float rate_;
};

// ------------------------------------------------------------------------------------------ device API
namespace cuda  // the reference's name for "the accelerator" (include/origin/cuda/cuda.h:25-105)
{
bool is_available();
int device_count();
int current_device();
void set_device(int device);
void device_info();
void synchronize();

// ---- beyond the reference (which queues everything on the null stream): a current stream per host thread, and a
// step recorded once and replayed. Usage: `void *s = cuda::create_stream(); cuda::set_stream(s);` run the step a few
// times (memory pool warm, optimizer buffers created), then `cuda::Graph g; g.begin_capture(); step(); g.end_capture();`
// and per iteration: `x.upload(batch); optimizer.prepare_replay(); g.launch();` — the tensors made by the capture run
// (the loss, the outputs) keep their addresses and hold the results of the latest replay. A captured step must not
// move data to or from the host (no item(), no to_vector(), no tensors built from host values): such a call throws.
// Memory allocated during the capture belongs to the graph until it is destroyed.
void *create_stream();
void destroy_stream(void *stream);
void set_stream(void *stream);  // nullptr = the null stream; synchronises the device when the stream changes
void *current_stream();
bool is_capturing();
// hands every cached block of the device memory pool that no tensor holds back to the driver (synchronises first)
void empty_cache();

class Graph
{
public:
    Graph() = default;
    ~Graph();
    Graph(const Graph &) = delete;
    Graph &operator=(const Graph &) = delete;
    void begin_capture();
    void end_capture();    // only the Graph that began the capture may end it
    void abort_capture();  // gives the capture up: the thread, its stream and the memory pool are as before begin_capture
    void launch();  // on the current stream
    bool captured() const { return exec_ != nullptr; }
    size_t node_count() const { return nodes_; }  // launches recorded

private:
    void *exec_ = nullptr;
    size_t nodes_ = 0;
    bool began_ = false;  // between this object's begin_capture and its end_capture / abort_capture
    std::shared_ptr<void> arena_;
};
}  // namespace cuda
}  // namespace origin
