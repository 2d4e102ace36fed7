// PNNX graph runner over the device backend. File formats as read by the reference (src/pnnx/pnnx_parser.cpp:36-380,
// src/pnnx/internal/store_zip.cpp:20-100); operator set as in src/pnnx/operator_mapper.cpp:26-78.
#include "origin/pnnx/pnnx_graph.h"

#include <cmath>
#include <cstdint>
#include <cstring>
#include <fstream>
#include <queue>
#include <sstream>

#include "origin/functional.h"
#include "origin/mat.h"

namespace origin
{
namespace pnnx
{
namespace
{
std::string trim(const std::string &s)
{
    const size_t a = s.find_first_not_of(" \t\r\n");
    if (a == std::string::npos)
        return "";
    return s.substr(a, s.find_last_not_of(" \t\r\n") - a + 1);
}

// "(1,3,6,6)f32" or "(2,2)" or "(2.0,2.0)" -> numbers between the parentheses
std::vector<double> numbers_in_parens(const std::string &v)
{
    std::vector<double> out;
    const size_t a = v.find('('), b = v.find(')');
    if (a == std::string::npos || b == std::string::npos || b < a)
        return out;
    std::stringstream ss(v.substr(a + 1, b - a - 1));
    std::string tok;
    while (std::getline(ss, tok, ','))
    {
        tok = trim(tok);
        if (tok.empty())
            continue;
        try
        {
            out.push_back(std::stod(tok));
        }
        catch (const std::exception &)
        {
            return {};  // not a numeric tuple (e.g. an expression)
        }
    }
    return out;
}

std::pair<int, int> int_pair(const PNNXNode &n, const std::string &key, std::pair<int, int> dflt)
{
    auto it = n.params.find(key);
    if (it == n.params.end())
        return dflt;
    const auto v = numbers_in_parens(it->second);
    if (v.size() >= 2)
        return {(int)v[0], (int)v[1]};
    if (v.size() == 1)
        return {(int)v[0], (int)v[0]};
    try
    {
        const int s = std::stoi(it->second);  // a bare integer
        return {s, s};
    }
    catch (const std::exception &)
    {
        return dflt;
    }
}

int int_param(const PNNXNode &n, const std::string &key, int dflt)
{
    auto it = n.params.find(key);
    if (it == n.params.end())
        return dflt;
    try
    {
        return std::stoi(it->second);
    }
    catch (const std::exception &)
    {
        return dflt;
    }
}

void parse_line(const std::string &line, PNNXNode &node)
{
    std::istringstream iss(line);
    int nin = 0, nout = 0;
    iss >> node.type >> node.name >> nin >> nout;
    if (!iss)
        THROW_RUNTIME_ERROR("PNNX param: malformed operator line '{}'", line);
    for (int i = 0; i < nin; ++i)
    {
        std::string s;
        iss >> s;
        node.input_names.push_back(s);
    }
    for (int i = 0; i < nout; ++i)
    {
        std::string s;
        iss >> s;
        node.output_names.push_back(s);
    }
    std::string tok;
    while (iss >> tok)
    {
        const size_t eq = tok.find('=');
        if (eq == std::string::npos || eq == 0)
            continue;
        const std::string key = tok.substr(0, eq), val = tok.substr(eq + 1);
        if (key[0] == '@')
        {
            Attribute a;
            for (double d : numbers_in_parens(val))
                a.shape.push_back((int)d);
            if (val.find("f32") == std::string::npos)
                THROW_RUNTIME_ERROR("PNNX param: attribute {} of node {} is not float32 ({})", key, node.name, val);
            node.attributes[key.substr(1)] = std::move(a);
        }
        else if (key[0] == '#')
        {
            std::vector<int> shp;
            for (double d : numbers_in_parens(val))
                shp.push_back((int)d);
            try
            {
                node.shapes[std::stoi(key.substr(1))] = shp;
            }
            catch (const std::exception &)
            {
                THROW_RUNTIME_ERROR("PNNX param: bad shape key '{}' in node {}", key, node.name);
            }
        }
        else
            node.params[key] = val;
    }
}

std::shared_ptr<Mat> upload(Attribute &a, const Device &dev, const std::string &who)
{
    if (a.device_mat && a.device_mat->device() == dev)
        return a.device_mat;
    if (a.data.empty() || a.shape.empty())
        THROW_RUNTIME_ERROR("PNNX: weight {} has no data (missing from the bin archive?)", who);
    std::vector<size_t> dims(a.shape.begin(), a.shape.end());
    a.device_mat = OriginMat::from_memory(a.data.data(), DataType::kFloat32, Shape(dims),
                                          TensorOptions(DataType::kFloat32).device(dev));
    return a.device_mat;
}

const OriginMat &origin_of(const Mat &m)
{
    const auto *o = dynamic_cast<const OriginMat *>(&m);
    if (!o)
        THROW_RUNTIME_ERROR("PNNX: expected an OriginMat, got backend_type={}", m.backend_type());
    return *o;
}
}  // namespace

std::map<std::string, std::vector<char>> read_store_zip(const std::string &path)
{
    std::ifstream f(path, std::ios::binary);
    if (!f.is_open())
        THROW_RUNTIME_ERROR("Failed to open bin file: {}", path);
    std::map<std::string, std::vector<char>> files;
    auto rd16 = [&](uint16_t &v) { f.read(reinterpret_cast<char *>(&v), 2); };
    auto rd32 = [&](uint32_t &v) { f.read(reinterpret_cast<char *>(&v), 4); };
    for (;;)
    {
        uint32_t sig = 0;
        rd32(sig);
        if (!f)
            break;
        if (sig == 0x04034b50u)  // local file header
        {
            uint16_t version, flag, compression, mtime, mdate, name_len, extra_len;
            uint32_t crc, csize, usize;
            rd16(version), rd16(flag), rd16(compression), rd16(mtime), rd16(mdate);
            rd32(crc), rd32(csize), rd32(usize);
            rd16(name_len), rd16(extra_len);
            if (!f || (flag & 0x08) || compression != 0 || csize != usize)
                THROW_RUNTIME_ERROR("{}: not a store-only zip archive (compressed or streamed member)", path);
            std::string name(name_len, '\0');
            f.read(&name[0], name_len);
            f.seekg(extra_len, std::ios::cur);
            std::vector<char> data(csize);
            f.read(data.data(), csize);
            if (!f)
                THROW_RUNTIME_ERROR("{}: truncated member {}", path, name);
            files[name] = std::move(data);
        }
        else if (sig == 0x02014b50u || sig == 0x06054b50u)
            break;  // central directory: every member has been seen
        else
            THROW_RUNTIME_ERROR("{}: unexpected record signature {}", path, sig);
    }
    return files;
}

PNNXGraph::PNNXGraph(const std::string &param_path, const std::string &bin_path)
    : param_path_(param_path), bin_path_(bin_path)
{}

void PNNXGraph::build()
{
    if (built_)
        return;
    if (param_path_.empty() || bin_path_.empty())
        THROW_RUNTIME_ERROR("Param path or bin path is empty");
    std::ifstream file(param_path_);
    if (!file.is_open())
        THROW_RUNTIME_ERROR("Failed to open param file: {}", param_path_);
    std::string line;
    std::getline(file, line);
    int magic = 0;
    try
    {
        magic = std::stoi(trim(line));
    }
    catch (const std::exception &)
    {
        THROW_RUNTIME_ERROR("Failed to parse magic number: '{}'", trim(line));
    }
    if (magic != 7767517)
        THROW_RUNTIME_ERROR("Invalid PNNX param file, magic number: {}", magic);
    std::getline(file, line);
    int op_count = 0, operand_count = 0;
    std::istringstream(line) >> op_count >> operand_count;
    nodes_.clear();
    for (int i = 0; i < op_count && std::getline(file, line); ++i)
    {
        if (trim(line).empty())
            continue;
        auto n = std::make_shared<PNNXNode>();
        parse_line(line, *n);
        nodes_.push_back(n);
    }
    if (nodes_.empty())
        THROW_RUNTIME_ERROR("Failed to parse PNNX model or model is empty");
    const auto files = read_store_zip(bin_path_);
    for (auto &n : nodes_)
    {
        by_name_[n->name] = n;
        for (auto &kv : n->attributes)
        {
            auto it = files.find(n->name + "." + kv.first);
            if (it == files.end())
                continue;
            size_t count = 1;
            for (int d : kv.second.shape)
                count *= (size_t)d;
            if (it->second.size() != count * sizeof(float))
                THROW_RUNTIME_ERROR("Weight file size mismatch for {}.{}: expected {} bytes, got {} bytes", n->name,
                                    kv.first, count * sizeof(float), it->second.size());
            kv.second.data.resize(count);
            std::memcpy(kv.second.data.data(), it->second.data(), it->second.size());
        }
    }
    // execution order: a node runs once everything it reads has a producer that ran (graph inputs count as ready)
    std::map<std::string, PNNXNode *> producer;
    for (auto &n : nodes_)
        for (auto &o : n->output_names)
            producer[o] = n.get();
    std::map<PNNXNode *, int> waiting;
    std::map<PNNXNode *, std::vector<PNNXNode *>> users;
    std::queue<PNNXNode *> ready;
    for (auto &n : nodes_)
    {
        int w = 0;
        for (auto &in : n->input_names)
        {
            auto it = producer.find(in);
            if (it == producer.end())
                THROW_RUNTIME_ERROR("PNNX: node {} reads '{}' that no node produces", n->name, in);
            if (it->second->type != "pnnx.Input")
            {
                ++w;
                users[it->second].push_back(n.get());
            }
        }
        waiting[n.get()] = w;
    }
    for (auto &n : nodes_)
        if (waiting[n.get()] == 0 && n->type != "pnnx.Input")
            ready.push(n.get());
    plan_.clear();
    int order = 0;
    while (!ready.empty())
    {
        PNNXNode *n = ready.front();
        ready.pop();
        n->execution_order = order++;
        if (n->type != "pnnx.Output")
            plan_.push_back(by_name_[n->name]);
        for (PNNXNode *u : users[n])
            if (--waiting[u] == 0)
                ready.push(u);
    }
    for (auto &n : nodes_)
        if (n->type != "pnnx.Input" && n->execution_order < 0)
            THROW_RUNTIME_ERROR("PNNX: node {} is part of a cycle", n->name);
    // conv -> activation pairs: the activation moves into the convolution's epilogue when nobody else reads the
    // convolution's output
    std::map<std::string, int> readers;
    for (auto &n : nodes_)
        for (auto &in : n->input_names)
            ++readers[in];
    for (auto &n : plan_)
    {
        if ((n->type != "nn.SiLU" && n->type != "nn.ReLU") || n->input_names.size() != 1 || n->output_names.size() != 1)
            continue;
        auto pit = producer.find(n->input_names[0]);
        if (pit == producer.end() || pit->second->type != "nn.Conv2d" || readers[n->input_names[0]] != 1 ||
            pit->second->output_names.size() != 1)
            continue;
        pit->second->fused_activation = n->type == "nn.SiLU" ? 7 : 0;
        pit->second->fused_output_name = n->output_names[0];
        n->folded_into_producer = true;
    }
    static const char *known[] = {"nn.Conv2d",  "nn.SiLU",        "nn.ReLU",   "nn.Upsample",        "nn.MaxPool2d", "pnnx.Expression",
                                  "torch.cat",  "torch.flatten", "nn.Linear", "models.yolo.Detect"};
    for (auto &n : plan_)
    {
        bool ok = false;
        for (const char *k : known)
            ok = ok || n->type == k;
        if (!ok)
            THROW_RUNTIME_ERROR("Unsupported operator type: {}", n->type);
    }
    built_ = true;
}

void PNNXGraph::set_inputs(const std::string &input_name, const std::vector<Tensor> &inputs)
{
    if (!built_)
        THROW_RUNTIME_ERROR("Graph must be built before setting inputs");
    auto it = by_name_.find(input_name);
    if (it == by_name_.end())
        THROW_RUNTIME_ERROR("Input node not found: {}", input_name);
    PNNXNode &n = *it->second;
    if (n.output_names.size() != inputs.size())
        THROW_RUNTIME_ERROR("Input count mismatch: input node has {} outputs, but {} inputs provided",
                            n.output_names.size(), inputs.size());
    for (size_t i = 0; i < inputs.size(); ++i)
        blobs_[n.output_names[i]] = inputs[i].impl_->data_;
}

void PNNXGraph::forward()
{
    if (!built_)
        THROW_RUNTIME_ERROR("Graph must be built before forward");
    for (auto &n : plan_)
        run(*n);
}

std::vector<Tensor> PNNXGraph::get_outputs(const std::string &output_name) const
{
    auto it = by_name_.find(output_name);
    if (it == by_name_.end())
        THROW_RUNTIME_ERROR("Output node not found: {}", output_name);
    std::vector<Tensor> out;
    for (auto &in : it->second->input_names)
    {
        auto b = blobs_.find(in);
        if (b == blobs_.end())
            THROW_RUNTIME_ERROR("Output '{}' has not been computed: call forward() first", in);
        out.emplace_back(std::make_shared<TensorImpl>(b->second));
    }
    return out;
}

void PNNXGraph::run(PNNXNode &node)
{
    if (node.folded_into_producer)
        return;  // its producer already wrote this node's output
    std::vector<std::shared_ptr<Mat>> in;
    for (auto &name : node.input_names)
    {
        auto it = blobs_.find(name);
        if (it == blobs_.end())
            THROW_RUNTIME_ERROR("PNNX: input '{}' of node {} has no value (set_inputs not called?)", name, node.name);
        in.push_back(it->second);
    }
    if (in.empty())
        THROW_RUNTIME_ERROR("PNNX: node {} ({}) has no inputs", node.name, node.type);
    const Device dev = in[0]->device();
    auto weight = [&](const std::string &key) -> std::shared_ptr<Mat> {
        auto it = node.attributes.find(key);
        if (it == node.attributes.end())
            return nullptr;
        return upload(it->second, dev, node.name + "." + key);
    };
    std::shared_ptr<Mat> out;
    const std::string &t = node.type;
    if (t == "nn.Conv2d")
    {
        if (int_pair(node, "dilation", {1, 1}) != std::make_pair(1, 1) || int_param(node, "groups", 1) != 1)
            THROW_RUNTIME_ERROR("PNNX: node {}: dilated or grouped convolutions are not supported", node.name);
        auto w = weight("weight");
        if (!w)
            THROW_RUNTIME_ERROR("PNNX: node {} has no weight", node.name);
        auto b = weight("bias");
        const auto stride = int_pair(node, "stride", {1, 1}), padding = int_pair(node, "padding", {0, 0});
        // the weights never change: the filter order this input shape's kernel wants is made once and kept
        Attribute &wa = node.attributes.find("weight")->second;
        const std::vector<size_t> in_dims = in[0]->shape().dims();
        if (wa.packed_for != in_dims)
        {
            wa.packed_mat = origin_of(*in[0]).conv2d_packed_weights(*w, stride, padding);
            wa.packed_for = in_dims;
        }
        out = origin_of(*in[0]).conv2d_act(*w, b.get(), stride, padding, node.fused_activation, wa.packed_mat.get());
    }
    else if (t == "nn.SiLU")
        out = in[0]->silu();
    else if (t == "nn.ReLU")
        out = in[0]->relu();
    else if (t == "nn.MaxPool2d")
    {
        const auto k = int_pair(node, "kernel_size", {2, 2});
        auto s = int_pair(node, "stride", {0, 0});
        if (s.first <= 0 || s.second <= 0)
            s = k;  // a missing stride means the kernel size
        out = in[0]->max_pool2d(k, s, int_pair(node, "padding", {0, 0}), nullptr);
    }
    else if (t == "nn.Upsample")
    {
        const Shape xs = in[0]->shape();
        if (xs.size() != 4)
            THROW_RUNTIME_ERROR("Upsample forward: x must be 4D (N, C, H, W), but got shape {}", xs.to_string());
        size_t OH, OW;
        const auto size = numbers_in_parens(node.params.count("size") ? node.params.at("size") : "");
        if (size.size() >= 2 && size[0] > 0 && size[1] > 0)
            OH = (size_t)size[0], OW = (size_t)size[1];
        else
        {
            auto sc = numbers_in_parens(node.params.count("scale_factor") ? node.params.at("scale_factor") : "");
            if (sc.empty())
                sc = {2.0, 2.0};  // the reference's default (operator_mapper.cpp:176-180)
            if (sc.size() == 1)
                sc.push_back(sc[0]);
            OH = (size_t)std::lround(xs[2] * sc[0]), OW = (size_t)std::lround(xs[3] * sc[1]);
        }
        const std::string mode = node.params.count("mode") ? node.params.at("mode") : "nearest";
        if (mode != "nearest")
            THROW_RUNTIME_ERROR("PNNX: node {}: upsample mode '{}' is not supported", node.name, mode);
        out = in[0]->upsample(Shape{xs[0], xs[1], OH, OW}, (int)(OH / xs[2]), (int)(OW / xs[3]), mode);
    }
    else if (t == "torch.cat")
    {
        std::vector<const Mat *> others;
        for (size_t i = 1; i < in.size(); ++i)
            others.push_back(in[i].get());
        out = in[0]->cat(others, int_param(node, "dim", 0));
    }
    else if (t == "pnnx.Expression")
    {
        const std::string expr = node.params.count("expr") ? node.params.at("expr") : "unknown";
        if (expr.find("add") == std::string::npos || in.size() != 2)
            THROW_RUNTIME_ERROR("Unsupported expression: {}", expr);
        out = *in[0] + *in[1];
    }
    else if (t == "torch.flatten")
    {
        const Shape xs = in[0]->shape();
        int a = int_param(node, "start_dim", 1), b = int_param(node, "end_dim", -1);
        const int nd = (int)xs.size();
        a = a < 0 ? a + nd : a, b = b < 0 ? b + nd : b;
        if (a < 0 || b >= nd || a > b)
            THROW_RUNTIME_ERROR("PNNX: node {}: bad flatten range [{}, {}] for {} dims", node.name, a, b, nd);
        std::vector<size_t> d;
        size_t prod = 1;
        for (int i = 0; i < nd; ++i)
        {
            if (i < a || i > b)
                d.push_back(xs[i]);
            else
            {
                prod *= xs[i];
                if (i == b)
                    d.push_back(prod);
            }
        }
        out = in[0]->reshape(Shape(d));
    }
    else if (t == "nn.Linear")
    {
        auto w = weight("weight");  // [out_features, in_features]
        if (!w)
            THROW_RUNTIME_ERROR("PNNX: node {} has no weight", node.name);
        auto wt = w->transpose();
        out = in[0]->matmul(*wt);
        if (auto b = weight("bias"))
            out = *out + *b->broadcast_to(out->shape());
    }
    else if (t == "models.yolo.Detect")
    {
        // attribute names as PNNX exports them for a three-stage head (operator_mapper.cpp:282-345):
        // strides pnnx_5; anchor grids pnnx_4/2/0 and grids pnnx_6/3/1 for stages 0/1/2; convolutions m.<stage>.{weight,bias}
        auto sit = node.attributes.find("pnnx_5");
        if (sit == node.attributes.end())
            THROW_RUNTIME_ERROR("YoloDetect: cannot find pnnx_5 (strides) attribute");
        const std::vector<float> &strides = sit->second.data;
        if (strides.size() != 3 || in.size() != 3)
            THROW_RUNTIME_ERROR("YoloDetect: only supports 3 stages, but got {} strides and {} inputs", strides.size(),
                                in.size());
        static const char *anchor_names[3] = {"pnnx_4", "pnnx_2", "pnnx_0"}, *grid_names[3] = {"pnnx_6", "pnnx_3", "pnnx_1"};
        std::vector<std::unique_ptr<Mat>> stages;
        for (int s = 0; s < 3; ++s)
        {
            auto w = weight("m." + std::to_string(s) + ".weight"), b = weight("m." + std::to_string(s) + ".bias");
            auto ag = weight(anchor_names[s]), g = weight(grid_names[s]);
            if (!w || !b || !ag || !g)
                THROW_RUNTIME_ERROR("YoloDetect: stage {} lacks one of weight / bias / anchor grid / grid", s);
            const int out_ch = (int)w->shape()[0];
            if (out_ch % 3 != 0 || out_ch / 3 - 5 <= 0)
                THROW_RUNTIME_ERROR("YoloDetect: out_channels ({}) must be 3 * (classes + 5)", out_ch);
            stages.push_back(in[s]->yolo_detect_forward(*w, b.get(), *g, *ag, strides[s], 3, out_ch / 3 - 5));
        }
        std::vector<const Mat *> others{stages[1].get(), stages[2].get()};
        out = stages[0]->cat(others, 1);
    }
    else
        THROW_RUNTIME_ERROR("Unsupported operator type: {}", t);
    if (node.output_names.size() != 1)
        THROW_RUNTIME_ERROR("PNNX: node {} declares {} outputs; this runner's operators produce one", node.name,
                            node.output_names.size());
    blobs_[node.fused_output_name.empty() ? node.output_names[0] : node.fused_output_name] = std::move(out);
}
}  // namespace pnnx
}  // namespace origin
