// Model files and checkpoints in the reference's own on-disk formats (include/origin/io/model_io.h, checkpoint.h;
// src/io/model_io.cpp:116-273, checkpoint.cpp:13-226), so that files written by either side load on the other.
//
// `.odl` (little-endian, size_t = 8 bytes): u32 magic 0x4F444C00 | u32 version 1 | u64 entry count | per entry:
// u64 name length + name bytes | u64 rank + u64 per dimension | i32 dtype | i32 device type + i32 device index |
// the elements, raw (float32, float64 or int32). A tensor is read back onto the device recorded in the file.
//
// A checkpoint `X.ckpt` is the directory `X/` holding `model.odl` and `metadata.json` (epoch, step, loss, optimizer
// type and the lr/beta1/beta2/eps settings, one per line). Optimizer buffers are not written, as in the reference.
#pragma once
#include <any>
#include <string>
#include <unordered_map>

#include "tensor.h"

namespace origin
{
using StateDict = std::unordered_map<std::string, Tensor>;

void save(const StateDict &state_dict, const std::string &filepath);
StateDict load(const std::string &filepath);

struct Checkpoint
{
    StateDict model_state_dict;
    std::unordered_map<std::string, std::unordered_map<std::string, std::any>> optimizer_state_dict;
    int epoch  = -1;
    int step   = -1;
    float loss = 0.0f;
    std::string optimizer_type;
    std::unordered_map<std::string, float> optimizer_config;
};

void save(const Checkpoint &checkpoint, const std::string &filepath);
Checkpoint load_checkpoint(const std::string &filepath);
}  // namespace origin
