// Internal to the library: the weight sources and the host-side random generator.
#pragma once
#include "../include/inference.h"

namespace tinyinfer {
std::unique_ptr<WeightSource> make_folder_source(const std::string& dir);
std::unique_ptr<WeightSource> make_tensors_source(const std::vector<HostTensor>& tensors, bool on_device);
std::unique_ptr<WeightSource> make_random_source(const std::vector<std::pair<std::string, TensorNeed>>& needs, uint64_t seed, Ops& ops);
void check_source(const std::string& where, const std::vector<std::pair<std::string, TensorNeed>>& needs, const WeightSource& src);
uint64_t tensor_seed(uint64_t seed, const std::string& name);
void host_random(const TensorNeed& need, uint64_t seed, DType dt, void* out);
}  // namespace tinyinfer
