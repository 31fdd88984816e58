// Drop-in C++ surface of the reference engine (Inference.cu:356-366): same
// class name, constructor and generateResponse signature, same weight
// directory, same failure behaviour (message on stderr, exit(1);
// Inference.cu:52-71, 299-308).  Everything behind it is the C ABI of
// awq_infer.h.
#pragma once
#include <string>
#include <vector>

struct awq_engine;

class QWen3AWQInfer {
 public:
  explicit QWen3AWQInfer(const std::string& weight_dir);
  ~QWen3AWQInfer();
  QWen3AWQInfer(const QWen3AWQInfer&) = delete;
  QWen3AWQInfer& operator=(const QWen3AWQInfer&) = delete;

  // prompt_ids: input token IDs; max_new_tokens: how many to generate;
  // returns only the newly generated token IDs (Inference.cu:361-366)
  std::vector<int> generateResponse(const std::vector<int>& prompt_ids, int max_new_tokens);

  // Not in the reference: send all prompt positions through each layer together
  // (one W4A16 matrix product per weight matrix instead of one matrix-vector
  // product per prompt token, Inference.cu:1304-1343).  Same state up to
  // binary16 rounding noise; off by default.
  void setBatchedPrefill(bool enabled);

 private:
  awq_engine* engine_;
};
