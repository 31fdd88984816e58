#include "qwen3_awq_infer.hpp"

#include <cstdlib>
#include <iostream>

#include "../../include/awq_infer.h"

static void die_on(int rc, const char* what) {
  if (rc == AWQ_OK) return;
  std::cerr << "ERROR: " << what << ": " << awq_last_error() << "\n";
  std::exit(1);
}

QWen3AWQInfer::QWen3AWQInfer(const std::string& weight_dir, PromptMode prompt_mode) : engine_(nullptr) {
  die_on(awq_create(weight_dir.c_str(), nullptr, &engine_), "QWen3AWQInfer");
  if (prompt_mode == PromptMode::Batched) setBatchedPrefill(true);
}

QWen3AWQInfer::~QWen3AWQInfer() { awq_destroy(engine_); }

std::vector<int> QWen3AWQInfer::generateResponse(const std::vector<int>& prompt_ids, int max_new_tokens) {
  std::vector<int32_t> prompt(prompt_ids.begin(), prompt_ids.end());
  std::vector<int32_t> out((size_t)(max_new_tokens > 0 ? max_new_tokens : 0));
  die_on(awq_generate(engine_, prompt.data(), (int32_t)prompt.size(), max_new_tokens, out.data()), "generateResponse");
  return std::vector<int>(out.begin(), out.end());
}

void QWen3AWQInfer::setBatchedPrefill(bool enabled) {
  die_on(awq_set_prefill_mode(engine_, enabled ? 1 : 0), "setBatchedPrefill");
}
