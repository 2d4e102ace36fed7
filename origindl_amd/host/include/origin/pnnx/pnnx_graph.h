// PNNX graph runner: loads a `.pnnx.param` / `.pnnx.bin` pair and runs it forward on the device backend.
// Same public surface as the reference's origin::pnnx::PNNXGraph (include/origin/pnnx/pnnx_graph.h:20-60):
// construct with the two paths, build(), set_inputs(name, tensors), forward(), get_outputs(name).
//
// Differences that do not change results: a convolution followed only by SiLU / ReLU runs as one kernel; weights are uploaded to the device once (at the first forward on that
// device) and kept, where the reference rebuilds every weight tensor from host data on every forward
// (src/pnnx/pnnx_graph.cpp:341-405); nodes run on Mat objects directly, without building an autograd graph.
#pragma once
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
    std::string fused_output_name;   // the activation node's output
    bool folded_into_producer = false;
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

private:
    std::string param_path_, bin_path_;
    std::vector<std::shared_ptr<PNNXNode>> nodes_, plan_;
    std::map<std::string, std::shared_ptr<PNNXNode>> by_name_;
    std::map<std::string, std::shared_ptr<Mat>> blobs_;  // tensor name -> value of the current forward
    bool built_ = false;
    void run(PNNXNode &node);
};

// store-only zip reader of the `.pnnx.bin` archive (src/pnnx/internal/store_zip.cpp:20-100 describes the format)
std::map<std::string, std::vector<char>> read_store_zip(const std::string &path);
}  // namespace pnnx
}  // namespace origin
