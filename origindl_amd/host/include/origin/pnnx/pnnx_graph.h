// PNNX graph runner: loads a `.pnnx.param` / `.pnnx.bin` pair and runs it forward on the device backend.
// Same public surface as the reference's origin::pnnx::PNNXGraph (include/origin/pnnx/pnnx_graph.h:20-60):
// construct with the two paths, build(), set_inputs(name, tensors), forward(), get_outputs(name).
//
// Differences that do not change what a node computes: a convolution followed only by SiLU / ReLU runs as one kernel,
// and so does the residual add that follows it alone; the inputs of a channel concatenation are written by their
// producers straight into the concatenation's output (and read from there by their other readers), so the torch.cat
// node copies only what could not be placed; a chain of same-size max pools whose stages are all concatenated (SPPF)
// is one launch; two convolutions that read the same tensor through the same window (the cv1 / cv2 pair of a C3 block)
// are one launch; the detect head decodes each stage into its rows of the final tensor. Weights are uploaded to the
// device once (at the first forward on that device) and kept, where the reference rebuilds every weight tensor from
// host data on every forward (src/pnnx/pnnx_graph.cpp:341-405); nodes run on Mat objects directly, without building
// an autograd graph. set_fusion(false) runs every node on its own, as the reference does.
#pragma once
#define ORIGINDL_AMD_PNNX_FUSION 1  // this runner has set_fusion()
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "../tensor.h"

namespace origin
{
namespace pnnx
{
struct Attribute  // a weight blob: `@name=(d0,d1,...)f32` in the param file, raw float32 in the bin archive
{
    std::vector<int> shape;
    std::vector<float> data;
    std::shared_ptr<Mat> device_mat;  // uploaded copy, created on first use
    // a convolution filter's re-ordered copy for inputs of shape packed_for (made on the first forward over that shape;
    // null when the forward reads the filter as it lies)
    std::shared_ptr<Mat> packed_mat;
    std::vector<size_t> packed_for;
};

struct PNNXNode
{
    std::string name, type;
    std::vector<std::string> input_names, output_names;
    std::map<std::string, std::string> params;  // raw text of every key=value that is neither @attribute nor #shape
    std::map<std::string, Attribute> attributes;
    std::map<int, std::vector<int>> shapes;
    int execution_order = -1;
    // set by build(): a convolution whose only reader is an activation applies it in its own epilogue and writes that
    // node's output; the activation node is then skipped
    int fused_activation = -1;       // -1 none, 0 relu, 7 silu
    std::string fused_output_name;   // the output of the last node folded into this one
    bool folded_into_producer = false;
    // a convolution that also performs the add that follows it: the add's other input
    std::string residual_name;
    // the first max pool of a chain of `pool_chain` same-size pools whose outputs lie side by side in one concatenation
    int pool_chain = 0;
    // a convolution that also runs the convolution `pair_with` (same input, window, stride, padding and activation):
    // the two filters follow each other in the attributes "pair.weight" / "pair.bias", made at the first forward
    std::string pair_with;
    // the node's numeric parameters, read out of `params` once (at the first forward)
    bool parsed = false;
    std::pair<int, int> kernel{1, 1}, stride{1, 1}, padding{0, 0};
};

class PNNXGraph
{
public:
    PNNXGraph(const std::string &param_path, const std::string &bin_path);
    void build();
    void set_inputs(const std::string &input_name, const std::vector<Tensor> &inputs);
    void forward();
    std::vector<Tensor> get_outputs(const std::string &output_name) const;

    // introspection used by tests and tools
    size_t node_count() const { return nodes_.size(); }
    const std::vector<std::shared_ptr<PNNXNode>> &execution_plan() const { return plan_; }
    // false: no node writes into another node's output and nothing is folded beyond conv + activation (call before
    // build()); the results are the same floats either way wherever the same convolution kernel runs
    void set_fusion(bool on) { fusion_ = on; }
    // nodes of the plan that launch work of their own in a forward (folded nodes do not)
    size_t launching_nodes() const;

private:
    // where a tensor of the current forward lives: a tensor of its own, or channels [c0, c0 + channels) of a
    // concatenation's output (`dense` then holds a copy of its own, made when a reader needs one)
    struct Value
    {
        std::shared_ptr<Mat> mat;
        size_t c0 = 0, channels = 0;
        bool run = false;
        std::shared_ptr<Mat> dense;
    };
    struct Placement  // decided by build(): this tensor is channels [c0, ...) of the torch.cat output `buffer`
    {
        std::string buffer;
        size_t c0 = 0;
    };
    std::string param_path_, bin_path_;
    std::vector<std::shared_ptr<PNNXNode>> nodes_, plan_;
    std::map<std::string, std::shared_ptr<PNNXNode>> by_name_;
    std::map<std::string, Value> blobs_;  // tensor name -> value of the current forward
    std::map<std::string, Placement> placed_;
    std::map<std::string, size_t> cat_channels_;  // torch.cat output -> its channel count, where build() could tell
    std::vector<std::string> input_blobs_;
    bool built_ = false, fusion_ = true;
    void run(PNNXNode &node);
    void run_conv(PNNXNode &node);
    void plan_fusion();
    Value destination(const std::string &tensor, size_t N, size_t C, size_t H, size_t W, const Device &dev);
    Value &value(const std::string &name, const PNNXNode &reader);
    std::shared_ptr<Mat> dense(const std::string &name, const PNNXNode &reader);
    std::shared_ptr<Mat> buffer_for(const std::string &cat_output, size_t N, size_t H, size_t W, const Device &dev);
    void store(const PNNXNode &node, std::shared_ptr<Mat> out);
};

// store-only zip reader of the `.pnnx.bin` archive (src/pnnx/internal/store_zip.cpp:20-100 describes the format)
std::map<std::string, std::vector<char>> read_store_zip(const std::string &path);
}  // namespace pnnx
}  // namespace origin
