// Host-side engine declarations shared by engine.cpp, synth.cpp and the C++
// wrapper class.
#pragma once
#include <string>
#include <vector>

#include "common.hpp"

// one file of the weight directory (Inference.cu:780-899)
struct WeightFile {
  std::string name;
  int layer, kind, part;
  int64_t bytes;
};

int awq_check_config(const awq_config* cfg);
std::vector<WeightFile> awq_weight_files(const awq_config& cfg);
// rows (outputs) and columns (inputs) of a quantised tensor kind
void awq_tensor_dims(const awq_config& cfg, int kind, int64_t* out_dim, int64_t* in_dim);
