// The reference's model-file and checkpoint formats, read and written from the host (src/io/model_io.cpp:116-273,
// src/io/checkpoint.cpp:13-226). Device tensors pass through one device-to-host or host-to-device copy each.
#include "origin/io.h"

#include <cstdint>
#include <cstdlib>
#include <filesystem>
#include <fstream>
#include <vector>

#include "origin/utils/exception.h"

namespace origin
{
namespace
{
constexpr uint32_t kMagic = 0x4F444C00;  // "ODL\0"
constexpr uint32_t kVersion = 1;

template <typename T>
void put(std::ofstream &out, const T &v)
{
    out.write(reinterpret_cast<const char *>(&v), sizeof(T));
}

template <typename T>
bool get(std::ifstream &in, T &v)
{
    in.read(reinterpret_cast<char *>(&v), sizeof(T));
    return !in.fail();
}

template <typename T>
void put_elements(std::ofstream &out, const Tensor &t)
{
    const std::vector<T> data = t.to_vector<T>();
    out.write(reinterpret_cast<const char *>(data.data()), (std::streamsize)(data.size() * sizeof(T)));
}

template <typename T>
Tensor get_elements(std::ifstream &in, const std::string &name, const Shape &shape, DataType dt, const Device &dev,
                    uint64_t bytes_left)
{
    const uint64_t n = shape.elements();
    if (n * sizeof(T) > bytes_left)  // a corrupt count must not turn into a huge allocation
        THROW_RUNTIME_ERROR("Failed to read tensor data for parameter '{}'", name);
    std::vector<T> data(n);
    in.read(reinterpret_cast<char *>(data.data()), (std::streamsize)(n * sizeof(T)));
    if (in.fail())
        THROW_RUNTIME_ERROR("Failed to read tensor data for parameter '{}'", name);
    return Tensor(data, shape, TensorOptions().dtype(dt).device(dev));
}

std::string checkpoint_dir(const std::string &filepath)
{
    if (filepath.size() > 5 && filepath.substr(filepath.size() - 5) == ".ckpt")
        return filepath.substr(0, filepath.size() - 5);
    return filepath;
}

// the text after the colon of a `"key": value` line, without blanks and the trailing comma
std::string json_value(const std::string &line)
{
    const size_t colon = line.find(':');
    if (colon == std::string::npos)
        return "";
    std::string v = line.substr(colon + 1);
    v.erase(0, v.find_first_not_of(" \t,"));
    v.erase(v.find_last_not_of(" \t,") + 1);
    return v;
}
}  // namespace

void save(const StateDict &state_dict, const std::string &filepath)
{
    std::ofstream out(filepath, std::ios::binary);
    if (!out.is_open())
        THROW_RUNTIME_ERROR("Failed to open file for writing: {}", filepath);
    put(out, kMagic);
    put(out, kVersion);
    put(out, (uint64_t)state_dict.size());
    for (const auto &[name, tensor] : state_dict)
    {
        put(out, (uint64_t)name.size());
        out.write(name.data(), (std::streamsize)name.size());
        const Shape shape = tensor.shape();
        put(out, (uint64_t)shape.size());
        for (size_t i = 0; i < shape.size(); ++i)
            put(out, (uint64_t)shape[i]);
        put(out, (int32_t)tensor.dtype());
        put(out, (int32_t)tensor.device().type());
        put(out, (int32_t)tensor.device().index());
        if (tensor.dtype() == DataType::kFloat32)
            put_elements<float>(out, tensor);
        else if (tensor.dtype() == DataType::kFloat64)
            put_elements<double>(out, tensor);
        else if (tensor.dtype() == DataType::kInt32)
            put_elements<int32_t>(out, tensor);
        else
            THROW_RUNTIME_ERROR("Unsupported dtype for saving: {}", static_cast<int>(tensor.dtype()));
    }
    out.close();
    if (out.fail())
        THROW_RUNTIME_ERROR("Failed to write to file: {}", filepath);
}

StateDict load(const std::string &filepath)
{
    std::ifstream in(filepath, std::ios::binary);
    if (!in.is_open())
        THROW_RUNTIME_ERROR("Failed to open file for reading: {}", filepath);
    in.seekg(0, std::ios::end);
    const uint64_t file_bytes = (uint64_t)in.tellg();
    in.seekg(0, std::ios::beg);
    uint32_t magic = 0, version = 0;
    if (!get(in, magic) || magic != kMagic)
        THROW_RUNTIME_ERROR("Invalid file format or corrupted file: {}", filepath);
    if (!get(in, version) || version != kVersion)
        THROW_RUNTIME_ERROR("Unsupported file version: {}", version);
    uint64_t count = 0;
    if (!get(in, count))
        THROW_RUNTIME_ERROR("Failed to read parameter count from file");
    StateDict state_dict;
    for (uint64_t i = 0; i < count; ++i)
    {
        uint64_t len = 0;
        if (!get(in, len) || len > file_bytes)
            THROW_RUNTIME_ERROR("Failed to read string length from file");
        std::string name(len, '\0');
        in.read(&name[0], (std::streamsize)len);
        if (in.fail())
            THROW_RUNTIME_ERROR("Failed to read string data from file");
        uint64_t rank = 0;
        if (!get(in, rank) || rank > 64)
            THROW_RUNTIME_ERROR("Failed to read shape dimensions from file");
        std::vector<size_t> dims(rank);
        for (uint64_t d = 0; d < rank; ++d)
        {
            uint64_t v = 0;
            if (!get(in, v))
                THROW_RUNTIME_ERROR("Failed to read shape dimension {} from file", d);
            dims[d] = (size_t)v;
        }
        const Shape shape(dims);
        int32_t dt = 0, dev_type = 0, dev_index = 0;
        if (!get(in, dt))
            THROW_RUNTIME_ERROR("Failed to read dtype from file");
        if (!get(in, dev_type) || !get(in, dev_index))
            THROW_RUNTIME_ERROR("Failed to read device from file");
        const DataType dtype = static_cast<DataType>(dt);
        const Device device(static_cast<DeviceType>(dev_type), dev_index);
        const uint64_t left = file_bytes - (uint64_t)in.tellg();
        Tensor tensor;
        if (dtype == DataType::kFloat32)
            tensor = get_elements<float>(in, name, shape, dtype, device, left);
        else if (dtype == DataType::kFloat64)
            tensor = get_elements<double>(in, name, shape, dtype, device, left);
        else if (dtype == DataType::kInt32)
            tensor = get_elements<int32_t>(in, name, shape, dtype, device, left);
        else
            THROW_RUNTIME_ERROR("Unsupported dtype for loading: {}", dt);
        state_dict[name] = tensor;
    }
    return state_dict;
}

void save(const Checkpoint &checkpoint, const std::string &filepath)
{
    namespace fs = std::filesystem;
    const std::string dir = checkpoint_dir(filepath);
    try
    {
        fs::create_directories(dir);
    }
    catch (const std::exception &e)
    {
        THROW_RUNTIME_ERROR("Failed to create checkpoint directory '{}': {}", dir, e.what());
    }
    save(checkpoint.model_state_dict, dir + "/model.odl");
    const std::string metadata_path = dir + "/metadata.json";
    std::ofstream meta(metadata_path);
    if (!meta.is_open())
        THROW_RUNTIME_ERROR("Failed to open metadata file for writing: {}", metadata_path);
    meta << "{\n";
    meta << "  \"format_version\": \"1.0\",\n";
    meta << "  \"format_type\": \"origindl_checkpoint\",\n";
    meta << "  \"epoch\": " << checkpoint.epoch << ",\n";
    meta << "  \"step\": " << checkpoint.step << ",\n";
    meta << "  \"loss\": " << checkpoint.loss << ",\n";
    meta << "  \"optimizer_type\": \"" << checkpoint.optimizer_type << "\",\n";
    meta << "  \"optimizer_config\": {\n";
    bool first = true;
    for (const auto &[key, value] : checkpoint.optimizer_config)
    {
        if (!first)
            meta << ",\n";
        meta << "    \"" << key << "\": " << value;
        first = false;
    }
    meta << "\n  }\n";
    meta << "}\n";
}

Checkpoint load_checkpoint(const std::string &filepath)
{
    namespace fs = std::filesystem;
    const std::string dir = checkpoint_dir(filepath);
    if (!fs::exists(dir) || !fs::is_directory(dir))
        THROW_RUNTIME_ERROR("Checkpoint directory does not exist: {}", dir);
    Checkpoint ck;
    const std::string model_path = dir + "/model.odl";
    if (!fs::exists(model_path))
        THROW_RUNTIME_ERROR("Model file not found in checkpoint: {}", model_path);
    ck.model_state_dict = load(model_path);
    const std::string metadata_path = dir + "/metadata.json";
    if (!fs::exists(metadata_path))
        THROW_RUNTIME_ERROR("Metadata file not found in checkpoint: {}", metadata_path);
    std::ifstream meta(metadata_path);
    if (!meta.is_open())
        THROW_RUNTIME_ERROR("Failed to open metadata file: {}", metadata_path);
    std::string line;
    while (std::getline(meta, line))
    {
        auto has = [&](const char *key) { return line.find(key) != std::string::npos; };
        if (has("\"epoch\""))
            ck.epoch = std::atoi(json_value(line).c_str());
        if (has("\"step\""))
            ck.step = std::atoi(json_value(line).c_str());
        if (has("\"loss\""))
            ck.loss = (float)std::atof(json_value(line).c_str());
        if (has("\"optimizer_type\""))
        {
            const size_t colon = line.find(':');
            if (colon != std::string::npos)
            {
                const std::string v = line.substr(colon + 1);
                const size_t a = v.find('"');
                const size_t b = a == std::string::npos ? a : v.find('"', a + 1);
                if (a != std::string::npos && b != std::string::npos)
                    ck.optimizer_type = v.substr(a + 1, b - a - 1);
            }
        }
        for (const char *key : {"lr", "beta1", "beta2", "eps"})
            if (has((std::string("\"") + key + "\"").c_str()))
                ck.optimizer_config[key] = (float)std::atof(json_value(line).c_str());
    }
    return ck;
}
}  // namespace origin
