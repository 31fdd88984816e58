// Drop-in C++ surface of the reference engine (Inference.cu:356-366): same
// class name, constructor and generateResponse signature, same weight
// directory, same failure behaviour (message on stderr, exit(1);
// Inference.cu:52-71, 299-308).  Everything behind it is the C ABI of
// awq_infer.h.
//
// One choice at construction: how generateResponse runs the PROMPT.
//   PromptMode::TokenByToken (default)  one forward pass per prompt token, as the
//       reference's loop does (Inference.cu:1304-1343); ids, hidden state and
//       logits are bit-identical to the CPU transcription.  A 128-token prompt
//       of the 36-layer model takes 128 ms on MI355X.
//   PromptMode::Batched  all prompt positions through each layer together (one
//       W4A16 matrix product per weight matrix): the same prompt in 4.2 ms, 31x
//       faster.  The state it leaves equals the other mode's up to binary16
//       rounding noise (products are summed in another order), so a greedy id
//       can differ where two logits are within that noise.
// Generation after the prompt is the same in both modes.
#pragma once
#include <string>
#include <vector>

struct awq_engine;

class QWen3AWQInfer {
 public:
  enum class PromptMode { TokenByToken, Batched };
  explicit QWen3AWQInfer(const std::string& weight_dir, PromptMode prompt_mode = PromptMode::TokenByToken);
  ~QWen3AWQInfer();
  QWen3AWQInfer(const QWen3AWQInfer&) = delete;
  QWen3AWQInfer& operator=(const QWen3AWQInfer&) = delete;

  // prompt_ids: input token IDs; max_new_tokens: how many to generate;
  // returns only the newly generated token IDs (Inference.cu:361-366)
  std::vector<int> generateResponse(const std::vector<int>& prompt_ids, int max_new_tokens);

  // the same choice after construction
  void setBatchedPrefill(bool enabled);

 private:
  awq_engine* engine_;
};
