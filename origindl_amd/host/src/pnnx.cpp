// PNNX graph runner over the device backend. File formats as read by the reference (src/pnnx/pnnx_parser.cpp:36-380,
// src/pnnx/internal/store_zip.cpp:20-100); operator set as in src/pnnx/operator_mapper.cpp:26-78.
#include "origin/pnnx/pnnx_graph.h"

#include <algorithm>
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

// (the weight's name is put together only for the error message: this runs for every weight of every node of every forward)
std::shared_ptr<Mat> upload(Attribute &a, const Device &dev, const std::string &node_name, const char *key)
{
    if (a.device_mat && a.device_mat->device() == dev)
        return a.device_mat;
    if (a.data.empty() || a.shape.empty())
        THROW_RUNTIME_ERROR("PNNX: weight {}.{} has no data (missing from the bin archive?)", node_name, key);
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
    placed_.clear();
    cat_channels_.clear();
    if (fusion_)
        plan_fusion();
    built_ = true;
}

namespace
{
// the tensor a node leaves behind once the nodes folded into it are counted in
const std::string &final_output(const PNNXNode &n)
{
    return n.fused_output_name.empty() ? n.output_names[0] : n.fused_output_name;
}

bool same_pool(const PNNXNode &n, int &K)
{
    if (n.type != "nn.MaxPool2d" || n.input_names.size() != 1 || n.output_names.size() != 1)
        return false;
    const auto k = int_pair(n, "kernel_size", {2, 2});
    auto s = int_pair(n, "stride", {0, 0});
    if (s.first <= 0 || s.second <= 0)
        s = k;
    const auto p = int_pair(n, "padding", {0, 0});
    K = k.first;
    return k.first == k.second && k.first % 2 == 1 && s == std::make_pair(1, 1) && p == std::make_pair(k.first / 2, k.first / 2);
}
}  // namespace

// Decides, from the graph alone, which adds fold into the convolution before them, which tensors are written
// straight into a concatenation's output, and which max pools form one chain. What a kernel can take is only known
// once the shapes are (at run time); a node that cannot honour a decision falls back to its own tensor and a copy.
void PNNXGraph::plan_fusion()
{
    std::map<std::string, PNNXNode *> writer;  // tensor -> the node that leaves it behind
    std::map<std::string, std::vector<PNNXNode *>> readers;
    for (auto &n : plan_)
    {
        if (!n->folded_into_producer && !n->output_names.empty())
            writer[final_output(*n)] = n.get();
        if (!n->folded_into_producer)
            for (auto &in : n->input_names)
                readers[in].push_back(n.get());
    }
    for (auto &n : nodes_)
        if (n->type == "pnnx.Output")
            for (auto &in : n->input_names)
                readers[in].push_back(n.get());
    // 1. conv (+ activation) -> add: the add moves into the convolution when the convolution's result has no other
    // reader and the other addend already exists when the convolution runs
    for (auto &n : plan_)
    {
        if (n->type != "pnnx.Expression" || n->input_names.size() != 2 || n->output_names.size() != 1)
            continue;
        const std::string expr = n->params.count("expr") ? n->params.at("expr") : "";
        if (expr.find("add") == std::string::npos || n->input_names[0] == n->input_names[1])
            continue;
        for (int side = 0; side < 2; ++side)
        {
            const std::string &t = n->input_names[side], &other = n->input_names[1 - side];
            auto w = writer.find(t);
            if (w == writer.end() || w->second->type != "nn.Conv2d" || !w->second->residual_name.empty() ||
                readers[t].size() != 1)
                continue;
            auto ow = writer.find(other);
            if (ow != writer.end() && ow->second->execution_order >= w->second->execution_order)
                continue;
            PNNXNode *conv = w->second;
            writer.erase(t);
            readers[other].push_back(conv);
            conv->residual_name = other;
            conv->fused_output_name = n->output_names[0];
            n->folded_into_producer = true;
            writer[n->output_names[0]] = conv;
            auto &ro = readers[other];
            ro.erase(std::remove(ro.begin(), ro.end(), n.get()), ro.end());
            break;
        }
    }
    // 1b. two convolutions that read the same tensor through the same window with the same activation run as one
    // launch over both filters (the later one folds into the earlier one)
    {
        auto same_params = [](const PNNXNode &a, const PNNXNode &b) {
            for (const char *key : {"kernel_size", "stride", "padding", "dilation", "groups", "padding_mode"})
            {
                const bool ha = a.params.count(key) > 0, hb = b.params.count(key) > 0;
                if (ha != hb || (ha && a.params.at(key) != b.params.at(key)))
                    return false;
            }
            auto wa = a.attributes.find("weight"), wb = b.attributes.find("weight");
            if (wa == a.attributes.end() || wb == b.attributes.end() || wa->second.shape.size() != 4 || wb->second.shape.size() != 4)
                return false;
            for (int d = 1; d < 4; ++d)
                if (wa->second.shape[d] != wb->second.shape[d])
                    return false;
            return (a.attributes.count("bias") > 0) == (b.attributes.count("bias") > 0);
        };
        for (size_t i = 0; i < plan_.size(); ++i)
        {
            PNNXNode &a = *plan_[i];
            if (a.type != "nn.Conv2d" || a.folded_into_producer || !a.pair_with.empty() || !a.residual_name.empty() ||
                a.input_names.size() != 1 || a.output_names.size() != 1)
                continue;
            for (size_t j = i + 1; j < plan_.size(); ++j)
            {
                PNNXNode &b = *plan_[j];
                if (b.type != "nn.Conv2d" || b.folded_into_producer || !b.pair_with.empty() || !b.residual_name.empty() ||
                    b.input_names != a.input_names || b.output_names.size() != 1 || b.fused_activation != a.fused_activation ||
                    !same_params(a, b))
                    continue;
                a.pair_with = b.name;
                b.folded_into_producer = true;
                break;
            }
        }
    }
    // 2. channel counts that follow from the graph alone
    std::map<std::string, size_t> channels;
    for (auto &n : plan_)
    {
        const bool paired_conv = n->folded_into_producer && n->type == "nn.Conv2d";  // runs inside its partner
        if ((n->folded_into_producer && !paired_conv) || n->output_names.size() != 1)
            continue;
        size_t c = 0;
        if (n->type == "nn.Conv2d")
        {
            auto w = n->attributes.find("weight");
            c = (w != n->attributes.end() && w->second.shape.size() == 4) ? (size_t)w->second.shape[0] : 0;
        }
        else if (n->type == "nn.SiLU" || n->type == "nn.ReLU" || n->type == "nn.MaxPool2d" || n->type == "nn.Upsample" ||
                 n->type == "pnnx.Expression")
            c = channels.count(n->input_names[0]) ? channels[n->input_names[0]] : 0;
        else if (n->type == "torch.cat" && int_param(*n, "dim", 0) == 1)
        {
            for (auto &in : n->input_names)
            {
                const size_t ci = channels.count(in) ? channels[in] : 0;
                if (ci == 0)
                {
                    c = 0;
                    break;
                }
                c += ci;
            }
        }
        if (c > 0)
            channels[final_output(*n)] = c;
    }
    // 3. inputs of a channel concatenation whose writer can aim at a run of channels are placed in its output
    for (auto &n : plan_)
    {
        if (n->type != "torch.cat" || int_param(*n, "dim", 0) != 1 || n->input_names.size() < 2 || n->output_names.size() != 1)
            continue;
        const std::string &out = n->output_names[0];
        if (!channels.count(out))
            continue;
        cat_channels_[out] = channels[out];
        size_t c0 = 0;
        for (auto &in : n->input_names)
        {
            auto w = writer.find(in);
            const bool can_aim = w != writer.end() && (w->second->type == "nn.Conv2d" || w->second->type == "nn.Upsample" ||
                                                       w->second->type == "nn.MaxPool2d");
            if (can_aim && !placed_.count(in))
                placed_[in] = Placement{out, c0};
            c0 += channels[in];
        }
    }
    // 4. chains of same-size max pools (stride 1, padding K/2) whose stages lie side by side in one concatenation
    for (auto &n : plan_)
    {
        int K = 0;
        if (n->folded_into_producer || !same_pool(*n, K) || !placed_.count(n->output_names[0]))
            continue;
        const Placement first = placed_[n->output_names[0]];
        const size_t C = channels.count(n->output_names[0]) ? channels[n->output_names[0]] : 0;
        if (C == 0)
            continue;
        int count = 1;
        PNNXNode *last = n.get();
        for (;;)
        {
            PNNXNode *next = nullptr;
            for (PNNXNode *r : readers[last->output_names[0]])
            {
                int K2 = 0;
                if (same_pool(*r, K2) && K2 == K && !r->folded_into_producer && r->pool_chain == 0)
                    next = r;
            }
            if (!next || !placed_.count(next->output_names[0]))
                break;
            const Placement &pl = placed_[next->output_names[0]];
            if (pl.buffer != first.buffer || pl.c0 != first.c0 + (size_t)count * C || count >= 8)
                break;
            next->folded_into_producer = true;
            ++count;
            last = next;
        }
        n->pool_chain = count;
    }
}

size_t PNNXGraph::launching_nodes() const
{
    size_t c = 0;
    for (auto &n : plan_)
        if (!n->folded_into_producer && n->type != "torch.flatten")
            ++c;
    return c;
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
    {
        Value v;
        v.mat = inputs[i].impl_->data_;
        blobs_[n.output_names[i]] = v;
        if (std::find(input_blobs_.begin(), input_blobs_.end(), n.output_names[i]) == input_blobs_.end())
            input_blobs_.push_back(n.output_names[i]);
    }
}

void PNNXGraph::forward()
{
    if (!built_)
        THROW_RUNTIME_ERROR("Graph must be built before forward");
    // the tensors of the previous forward go (a concatenation's output is made when its first input is written, so
    // one left over from the last forward must not be mistaken for it)
    for (auto it = blobs_.begin(); it != blobs_.end();)
    {
        if (std::find(input_blobs_.begin(), input_blobs_.end(), it->first) == input_blobs_.end())
            it = blobs_.erase(it);
        else
            ++it;
    }
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
        if (b == blobs_.end() || !b->second.mat)
            THROW_RUNTIME_ERROR("Output '{}' has not been computed: call forward() first", in);
        const Value &v = b->second;
        if (!v.run)
            out.emplace_back(std::make_shared<TensorImpl>(v.mat));
        else
        {
            // a graph output that lives inside a concatenation: handed out as a tensor of its own
            const Shape bs = v.mat->shape();
            std::shared_ptr<Mat> copy = std::make_shared<OriginMat>(Shape{bs[0], v.channels, bs[2], bs[3]}, DataType::kFloat32, v.mat->device());
            OriginMat::copy_run(OriginMat::ChannelRun{&origin_of(*v.mat), v.c0, v.channels}, OriginMat::whole(*copy));
            out.emplace_back(std::make_shared<TensorImpl>(copy));
        }
    }
    return out;
}

PNNXGraph::Value &PNNXGraph::value(const std::string &name, const PNNXNode &reader)
{
    auto it = blobs_.find(name);
    if (it == blobs_.end() || !it->second.mat)
        THROW_RUNTIME_ERROR("PNNX: input '{}' of node {} has no value (set_inputs not called?)", name, reader.name);
    return it->second;
}

// the tensor as one of its own: a run of channels inside a concatenation is copied out once, when first asked for
std::shared_ptr<Mat> PNNXGraph::dense(const std::string &name, const PNNXNode &reader)
{
    Value &v = value(name, reader);
    if (!v.run)
        return v.mat;
    if (!v.dense)
    {
        const Shape bs = v.mat->shape();
        v.dense = std::make_shared<OriginMat>(Shape{bs[0], v.channels, bs[2], bs[3]}, DataType::kFloat32, v.mat->device());
        OriginMat::copy_run(OriginMat::ChannelRun{&origin_of(*v.mat), v.c0, v.channels}, OriginMat::whole(*v.dense));
    }
    return v.dense;
}

std::shared_ptr<Mat> PNNXGraph::buffer_for(const std::string &cat_output, size_t N, size_t H, size_t W, const Device &dev)
{
    Value &v = blobs_[cat_output];
    const Shape want{N, cat_channels_.at(cat_output), H, W};
    if (!v.mat)
        v.mat = std::make_shared<OriginMat>(want, DataType::kFloat32, dev);
    else if (v.mat->shape() != want)
        THROW_RUNTIME_ERROR("PNNX: inputs of the concatenation {} disagree about its shape ({} and {})", cat_output,
                            v.mat->shape().to_string(), want.to_string());
    return v.mat;
}

// a node's dense result: kept as it is, or — for a tensor that build() placed in a concatenation — copied to its place
void PNNXGraph::store(const PNNXNode &node, std::shared_ptr<Mat> out)
{
    const std::string &name = final_output(node);
    auto pl = placed_.find(name);
    const Shape os = out->shape();
    if (pl == placed_.end() || os.size() != 4 || out->dtype() != DataType::kFloat32)
    {
        if (pl != placed_.end())
            placed_.erase(pl);  // not a 4D float tensor after all: the concatenation copies it like any other input
        Value v;
        v.mat = std::move(out);
        blobs_[name] = v;
        return;
    }
    auto buf = buffer_for(pl->second.buffer, os[0], os[2], os[3], out->device());
    OriginMat::copy_run(OriginMat::whole(*out), OriginMat::ChannelRun{&origin_of(*buf), pl->second.c0, os[1]});
    Value v;
    v.mat = buf, v.c0 = pl->second.c0, v.channels = os[1], v.run = true, v.dense = std::move(out);
    blobs_[name] = v;
}

// where a [N, C, H, W] tensor goes: its run of the concatenation build() placed it in, or a tensor of its own
PNNXGraph::Value PNNXGraph::destination(const std::string &tensor, size_t N, size_t C, size_t H, size_t W, const Device &dev)
{
    Value v;
    auto place = placed_.find(tensor);
    if (place != placed_.end())
    {
        v.mat = buffer_for(place->second.buffer, N, H, W, dev);
        v.c0 = place->second.c0, v.channels = C, v.run = true;
    }
    else
        v.mat = std::make_shared<OriginMat>(Shape{N, C, H, W}, DataType::kFloat32, dev);
    return v;
}

void PNNXGraph::run_conv(PNNXNode &node)
{
    Value &first = value(node.input_names[0], node);
    const Device dev = first.mat->device();
    auto run_of = [&](const Value &v) {
        return v.run ? OriginMat::ChannelRun{&origin_of(*v.mat), v.c0, v.channels} : OriginMat::whole(*v.mat);
    };
    if (!node.parsed)
    {
        if (int_pair(node, "dilation", {1, 1}) != std::make_pair(1, 1) || int_param(node, "groups", 1) != 1)
            THROW_RUNTIME_ERROR("PNNX: node {}: dilated or grouped convolutions are not supported", node.name);
        node.stride = int_pair(node, "stride", {1, 1}), node.padding = int_pair(node, "padding", {0, 0});
        node.parsed = true;
    }
    auto wit = node.attributes.find("weight");
    if (wit == node.attributes.end())
        THROW_RUNTIME_ERROR("PNNX: node {} has no weight", node.name);
    auto w = upload(wit->second, dev, node.name, "weight");
    auto bit = node.attributes.find("bias");
    std::shared_ptr<Mat> b = bit == node.attributes.end() ? nullptr : upload(bit->second, dev, node.name, "bias");
    const auto stride = node.stride, padding = node.padding;
    const Shape s0 = first.mat->shape();
    const Shape xs = (first.run && s0.size() == 4) ? Shape{s0[0], first.channels, s0[2], s0[3]} : s0;
    const Shape ws = w->shape();
    const bool f32 = first.mat->dtype() == DataType::kFloat32;
    const std::string &out_name = final_output(node);
    // this convolution and the one paired with it as one launch over both filters
    if (!node.pair_with.empty())
    {
        PNNXNode &other = *by_name_.at(node.pair_with);
        auto owit = other.attributes.find("weight");
        auto ow = upload(owit->second, dev, other.name, "weight");
        const Shape ows = ow->shape();
        const Shape both{ws[0] + ows[0], ws[1], ws[2], ws[3]};
        if (fusion_ && f32 && xs.size() == 4 && OriginMat::conv2d_fused_ok(xs, both, stride, padding))
        {
            Attribute &pw = node.attributes["pair.weight"];
            if (!pw.device_mat || pw.device_mat->device() != dev)
            {
                pw.device_mat = w->cat({ow.get()}, 0);
                pw.packed_for.clear();
                if (b)
                {
                    auto ob = upload(other.attributes.find("bias")->second, dev, other.name, "bias");
                    node.attributes["pair.bias"].device_mat = b->cat({ob.get()}, 0);
                }
            }
            if (pw.packed_for != xs.dims())
            {
                pw.packed_mat = OriginMat::conv2d_packed_weights_for(xs, *pw.device_mat, stride, padding);
                pw.packed_for = xs.dims();
            }
            if (pw.packed_mat)
            {
                const int OH = get_conv_outsize((int)xs[2], (int)ws[2], stride.first, padding.first);
                const int OW = get_conv_outsize((int)xs[3], (int)ws[3], stride.second, padding.second);
                const std::string &other_out = final_output(other);
                Value out = destination(out_name, xs[0], ws[0], (size_t)OH, (size_t)OW, dev);
                Value out2 = destination(other_out, xs[0], ows[0], (size_t)OH, (size_t)OW, dev);
                OriginMat::conv2d_fused_pair(run_of(first), *pw.packed_mat, both, b ? node.attributes["pair.bias"].device_mat.get() : nullptr,
                                             stride, padding, node.fused_activation, run_of(out), run_of(out2));
                blobs_[out_name] = out;
                blobs_[other_out] = out2;
                return;
            }
        }
    }
    // the weights never change: the filter order this input shape's kernel wants is made once and kept
    Attribute &wa = wit->second;
    if (wa.packed_for != xs.dims())
    {
        wa.packed_mat = OriginMat::conv2d_packed_weights_for(xs, *w, stride, padding);
        wa.packed_for = xs.dims();
    }
    if (fusion_ && wa.packed_mat && f32 && OriginMat::conv2d_fused_ok(xs, ws, stride, padding))
    {
        const int OH = get_conv_outsize((int)xs[2], (int)ws[2], stride.first, padding.first);
        const int OW = get_conv_outsize((int)xs[3], (int)ws[3], stride.second, padding.second);
        Value out = destination(out_name, xs[0], ws[0], (size_t)OH, (size_t)OW, dev);
        OriginMat::ChannelRun res{};
        if (!node.residual_name.empty())
            res = run_of(value(node.residual_name, node));
        OriginMat::conv2d_fused(run_of(first), *wa.packed_mat, ws, b.get(), stride, padding, node.fused_activation,
                                node.residual_name.empty() ? nullptr : &res, run_of(out));
        blobs_[out_name] = out;
    }
    else
    {
        auto x = dense(node.input_names[0], node);
        std::shared_ptr<Mat> out = origin_of(*x).conv2d_act(*w, b.get(), stride, padding, node.fused_activation, wa.packed_mat.get());
        if (!node.residual_name.empty())
            out = *dense(node.residual_name, node) + *out;
        store(node, std::move(out));
    }
    if (!node.pair_with.empty())
        run_conv(*by_name_.at(node.pair_with));  // the pair could not run as one: the partner on its own
}

void PNNXGraph::run(PNNXNode &node)
{
    if (node.folded_into_producer)
        return;  // its producer already wrote this node's output
    if (node.input_names.empty())
        THROW_RUNTIME_ERROR("PNNX: node {} ({}) has no inputs", node.name, node.type);
    if (node.output_names.size() != 1)
        THROW_RUNTIME_ERROR("PNNX: node {} declares {} outputs; this runner's operators produce one", node.name,
                            node.output_names.size());
    Value &first = value(node.input_names[0], node);
    const Device dev = first.mat->device();
    auto weight = [&](const std::string &key) -> std::shared_ptr<Mat> {
        auto it = node.attributes.find(key);
        if (it == node.attributes.end())
            return nullptr;
        return upload(it->second, dev, node.name, key.c_str());
    };
    auto run_of = [&](const Value &v) {
        return v.run ? OriginMat::ChannelRun{&origin_of(*v.mat), v.c0, v.channels} : OriginMat::whole(*v.mat);
    };
    auto run_shape = [&](const Value &v) {
        const Shape s = v.mat->shape();
        return (v.run && s.size() == 4) ? Shape{s[0], v.channels, s[2], s[3]} : s;
    };
    const std::string &out_name = final_output(node);
    auto place = placed_.find(out_name);
    const std::string &t = node.type;
    if (t == "nn.Conv2d")
    {
        run_conv(node);
        return;
    }
    if (t == "nn.MaxPool2d")
    {
        if (!node.parsed)
        {
            node.kernel = int_pair(node, "kernel_size", {2, 2});
            node.stride = int_pair(node, "stride", {0, 0});
            if (node.stride.first <= 0 || node.stride.second <= 0)
                node.stride = node.kernel;  // a missing stride means the kernel size
            node.padding = int_pair(node, "padding", {0, 0});
            node.parsed = true;
        }
        const auto k = node.kernel, s = node.stride;
        const Shape xs = run_shape(first);
        // this pool and the pools folded into it, in order
        std::vector<PNNXNode *> stages{&node};
        for (int j = 1; j < node.pool_chain; ++j)
            for (auto &n : plan_)
                if (n->folded_into_producer && n->type == "nn.MaxPool2d" && n->input_names[0] == stages.back()->output_names[0])
                {
                    stages.push_back(n.get());
                    break;
                }
        if ((int)stages.size() != (node.pool_chain > 0 ? node.pool_chain : 1))
            THROW_RUNTIME_ERROR("PNNX: node {}: the chain of {} max pools planned at build() is not in the graph", node.name,
                                node.pool_chain);
        if (node.pool_chain > 0 && place != placed_.end() && xs.size() == 4 && first.mat->dtype() == DataType::kFloat32 &&
            xs[2] * xs[3] <= 8192 && k.first <= 15)
        {
            // stage j goes to channels [c0 + (j-1)*C, c0 + j*C) of the concatenation: one launch for the whole chain
            auto buf = buffer_for(place->second.buffer, xs[0], xs[2], xs[3], dev);
            OriginMat::max_pool_chain(run_of(first), k.first, node.pool_chain,
                                      OriginMat::ChannelRun{&origin_of(*buf), place->second.c0, xs[1] * (size_t)node.pool_chain});
            for (size_t j = 0; j < stages.size(); ++j)
            {
                Value v;
                v.mat = buf, v.c0 = place->second.c0 + j * xs[1], v.channels = xs[1], v.run = true;
                blobs_[stages[j]->output_names[0]] = v;
            }
            return;
        }
        // one pool after the other, each result copied to its place
        for (PNNXNode *stage : stages)
            store(*stage, dense(stage->input_names[0], *stage)->max_pool2d(k, s, node.padding, nullptr));
        return;
    }
    if (t == "nn.Upsample")
    {
        const Shape xs = run_shape(first);
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
        const int sh = (int)(OH / xs[2]), sw = (int)(OW / xs[3]);
        if ((first.run || place != placed_.end()) && first.mat->dtype() == DataType::kFloat32 && OW % 4 == 0 && sh > 0 && sw > 0)
        {
            Value out = destination(out_name, xs[0], xs[1], OH, OW, dev);
            OriginMat::upsample_run(run_of(first), run_of(out), sh, sw);
            blobs_[out_name] = out;
            return;
        }
        std::shared_ptr<Mat> out = dense(node.input_names[0], node)->upsample(Shape{xs[0], xs[1], OH, OW}, sh, sw, mode);
        store(node, std::move(out));
        return;
    }
    if (t == "torch.cat")
    {
        const int dim = int_param(node, "dim", 0);
        auto cc = cat_channels_.find(node.output_names[0]);
        bool any_placed = false;
        for (auto &in : node.input_names)
        {
            auto pl = placed_.find(in);
            any_placed = any_placed || (pl != placed_.end() && pl->second.buffer == node.output_names[0]);
        }
        if (cc != cat_channels_.end() && any_placed)
        {
            // the output exists already, with the placed inputs in it; the others are copied to their channels
            std::shared_ptr<Mat> buf;
            size_t c0 = 0;
            for (auto &in : node.input_names)
            {
                Value &v = value(in, node);
                const Shape s = run_shape(v);
                if (s.size() != 4)
                    THROW_RUNTIME_ERROR("PNNX: node {}: input {} is not 4D", node.name, in);
                if (!buf)
                    buf = buffer_for(node.output_names[0], s[0], s[2], s[3], dev);
                const bool in_place = v.run && v.mat == buf && v.c0 == c0;
                if (!in_place)
                    OriginMat::copy_run(run_of(v), OriginMat::ChannelRun{&origin_of(*buf), c0, s[1]});
                c0 += s[1];
            }
            if (c0 != cc->second)
                THROW_RUNTIME_ERROR("PNNX: node {}: the inputs hold {} channels, the plan expected {}", node.name, c0, cc->second);
            return;  // blobs_[output] is the buffer
        }
        std::vector<std::shared_ptr<Mat>> in;
        for (auto &name : node.input_names)
            in.push_back(dense(name, node));
        std::vector<const Mat *> others;
        for (size_t i = 1; i < in.size(); ++i)
            others.push_back(in[i].get());
        store(node, in[0]->cat(others, dim));
        return;
    }
    if (t == "models.yolo.Detect")
    {
        // attribute names as PNNX exports them for a three-stage head (operator_mapper.cpp:282-345):
        // strides pnnx_5; anchor grids pnnx_4/2/0 and grids pnnx_6/3/1 for stages 0/1/2; convolutions m.<stage>.{weight,bias}
        auto sit = node.attributes.find("pnnx_5");
        if (sit == node.attributes.end())
            THROW_RUNTIME_ERROR("YoloDetect: cannot find pnnx_5 (strides) attribute");
        const std::vector<float> &strides = sit->second.data;
        if (strides.size() != 3 || node.input_names.size() != 3)
            THROW_RUNTIME_ERROR("YoloDetect: only supports 3 stages, but got {} strides and {} inputs", strides.size(),
                                node.input_names.size());
        static const char *anchor_names[3] = {"pnnx_4", "pnnx_2", "pnnx_0"}, *grid_names[3] = {"pnnx_6", "pnnx_3", "pnnx_1"};
        std::shared_ptr<Mat> ws[3], bs[3], ags[3], gs[3];
        size_t rows = 0, ci = 0;
        bool direct = fusion_;
        for (int s = 0; s < 3; ++s)
        {
            ws[s] = weight("m." + std::to_string(s) + ".weight"), bs[s] = weight("m." + std::to_string(s) + ".bias");
            ags[s] = weight(anchor_names[s]), gs[s] = weight(grid_names[s]);
            if (!ws[s] || !bs[s] || !ags[s] || !gs[s])
                THROW_RUNTIME_ERROR("YoloDetect: stage {} lacks one of weight / bias / anchor grid / grid", s);
            const int out_ch = (int)ws[s]->shape()[0];
            if (out_ch % 3 != 0 || out_ch / 3 - 5 <= 0)
                THROW_RUNTIME_ERROR("YoloDetect: out_channels ({}) must be 3 * (classes + 5)", out_ch);
            const Shape xs = run_shape(value(node.input_names[s], node));
            direct = direct && xs.size() == 4 && (ci == 0 || ci == (size_t)out_ch / 3);
            ci = (size_t)out_ch / 3;
            if (xs.size() == 4)
                rows += 3 * xs[2] * xs[3];
        }
        if (direct)
        {
            // the stages' 1x1 convolutions, then their decoding straight into each stage's rows of the final tensor
            const size_t N = run_shape(first)[0];
            std::shared_ptr<Mat> out = std::make_shared<OriginMat>(Shape{N, rows, ci}, DataType::kFloat32, dev);
            std::shared_ptr<Mat> convs[3];
            std::vector<Shape> xshapes, wshapes;
            bool packed_all = true;
            for (int s = 0; s < 3; ++s)
            {
                const Shape xs = run_shape(value(node.input_names[s], node));
                Attribute &wa = node.attributes.find("m." + std::to_string(s) + ".weight")->second;
                if (wa.packed_for != xs.dims())
                {
                    wa.packed_mat = OriginMat::conv2d_packed_weights_for(xs, *ws[s], {1, 1}, {0, 0});
                    wa.packed_for = xs.dims();
                }
                packed_all = packed_all && wa.packed_mat;
                xshapes.push_back(xs), wshapes.push_back(ws[s]->shape());
            }
            if (packed_all && OriginMat::yolo_detect_stages_ok(xshapes, 3, (int)ci - 5))
            {
                // (the stages do not depend on each other and each is a launch's latency long: one launch for the three
                // convolutions, which decode their sums themselves)
                std::vector<OriginMat::ChannelRun> xr;
                std::vector<const Mat *> pk, bv;
                for (int s = 0; s < 3; ++s)
                {
                    xr.push_back(run_of(value(node.input_names[s], node)));
                    pk.push_back(node.attributes.find("m." + std::to_string(s) + ".weight")->second.packed_mat.get());
                    bv.push_back(bs[s].get());
                }
                OriginMat::yolo_detect_stages(xr, pk, bv, {gs[0].get(), gs[1].get(), gs[2].get()},
                                              {ags[0].get(), ags[1].get(), ags[2].get()}, strides, 3, (int)ci - 5, *out);
                store(node, std::move(out));
                return;
            }
            // (a head the one launch does not take: stage by stage, then one launch that decodes the three)
            for (int s = 0; s < 3; ++s)
            {
                Value &xv = value(node.input_names[s], node);
                const Shape &xs = xshapes[s], &wsh = wshapes[s];
                Attribute &wa = node.attributes.find("m." + std::to_string(s) + ".weight")->second;
                if (wa.packed_mat && OriginMat::conv2d_fused_ok(xs, wsh, {1, 1}, {0, 0}))
                {
                    convs[s] = std::make_shared<OriginMat>(Shape{xs[0], wsh[0], xs[2], xs[3]}, DataType::kFloat32, dev);
                    OriginMat::conv2d_fused(run_of(xv), *wa.packed_mat, wsh, bs[s].get(), {1, 1}, {0, 0}, -1, nullptr,
                                            OriginMat::whole(*convs[s]));
                }
                else
                    convs[s] = origin_of(*dense(node.input_names[s], node)).conv2d_act(*ws[s], bs[s].get(), {1, 1}, {0, 0}, -1, wa.packed_mat.get());
            }
            // (one launch for the three stages: each is a chain of a load, sigmoids and a store, shorter than a launch)
            OriginMat::yolo_decode_stages_into({convs[0].get(), convs[1].get(), convs[2].get()}, {gs[0].get(), gs[1].get(), gs[2].get()},
                                               {ags[0].get(), ags[1].get(), ags[2].get()}, strides, 3, (int)ci - 5, *out);
            store(node, std::move(out));
            return;
        }
        std::vector<std::unique_ptr<Mat>> stages;
        for (int s = 0; s < 3; ++s)
            stages.push_back(dense(node.input_names[s], node)->yolo_detect_forward(*ws[s], bs[s].get(), *gs[s], *ags[s], strides[s], 3,
                                                                                  (int)ws[s]->shape()[0] / 3 - 5));
        std::vector<const Mat *> others{stages[1].get(), stages[2].get()};
        store(node, stages[0]->cat(others, 1));
        return;
    }
    // the remaining operators work on tensors of their own
    std::vector<std::shared_ptr<Mat>> in;
    for (auto &name : node.input_names)
        in.push_back(dense(name, node));
    std::shared_ptr<Mat> out;
    if (t == "nn.SiLU")
        out = in[0]->silu();
    else if (t == "nn.ReLU")
        out = in[0]->relu();
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
    else
        THROW_RUNTIME_ERROR("Unsupported operator type: {}", t);
    store(node, std::move(out));
}
}  // namespace pnnx
}  // namespace origin
