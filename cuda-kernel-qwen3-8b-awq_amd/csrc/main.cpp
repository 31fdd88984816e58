// Command-line harness with the behaviour of the reference's main
// (Inference.cu:1413-1433): one argument, BOS prompt, 20 greedy tokens.
#include <iostream>
#include <string>
#include <vector>

#include "qwen3_awq_infer.hpp"

int main(int argc, char** argv) {
  if (argc < 2) {
    std::cerr << "Usage: " << argv[0] << " <path_to_weight_folder>\n";
    return 1;
  }
  std::string weight_dir = argv[1];
  QWen3AWQInfer infer(weight_dir);

  std::vector<int> prompt = {151643};
  int max_new_tokens = 20;
  std::vector<int> out = infer.generateResponse(prompt, max_new_tokens);

  std::cout << "Generated tokens: ";
  for (int tok : out) std::cout << tok << " ";
  std::cout << std::endl;
  return 0;
}
