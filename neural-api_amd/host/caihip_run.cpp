// Command-line twin of the reference's greedy decode loop (TChatEngine.GenerateFromIds,
// neural/neuralchatengine.pas:1428-1561, greedy branch 1493-1494; --stats timing 1590-1605) over token ids:
//   caihip_run MODEL.gguf N_NEW [--max-ctx N] [--stepwise] TOKEN_ID...
// Prefills the prompt, then decodes N_NEW tokens greedily and prints them on one line; a second line reports the
// prompt and decode rates the way --stats does (tokens / (t_end - t_first)).  Tokenisation stays with the caller.
#include "caihip_host.hpp"

#include <chrono>
#include <cstdlib>
#include <cstring>

int main(int argc, char** argv)
{
  if (argc < 4) { std::fprintf(stderr, "usage: %s MODEL.gguf N_NEW [--max-ctx N] [--stepwise] TOKEN_ID...\n", argv[0]); return 2; }
  const std::string model = argv[1];
  const int n_new = std::atoi(argv[2]);
  int max_ctx = 0; bool stepwise = false;
  std::vector<int32_t> prompt;
  for (int i = 3; i < argc; i++) {
    if (!std::strcmp(argv[i], "--max-ctx") && i + 1 < argc) max_ctx = std::atoi(argv[++i]);
    else if (!std::strcmp(argv[i], "--stepwise")) stepwise = true;
    else prompt.push_back((int32_t)std::atoi(argv[i]));
  }
  if (prompt.empty() || n_new < 1) { std::fprintf(stderr, "need at least one prompt token and N_NEW >= 1\n"); return 2; }
  try {
    caihip::EnableHIP(0);
    caihip::TNNetStreamingDecoder dec(model, max_ctx);
    using clk = std::chrono::steady_clock;
    const auto t0 = clk::now();
    dec.Reset();
    if (stepwise) for (size_t i = 0; i < prompt.size(); i++) dec.StepForward(&prompt[i], 1, (int)i);
    else dec.StepForward(prompt.data(), (int)prompt.size(), 0);
    const auto t1 = clk::now();
    std::vector<int32_t> out;
    out.push_back(dec.ArgMaxRow());
    if (n_new > 1) {
      if (stepwise) {
        for (int k = 1; k < n_new; k++) { const int32_t t = out.back(); dec.StepForward(&t, 1, (int)prompt.size() + k - 1); out.push_back(dec.ArgMaxRow()); }
      } else {
        const std::vector<int32_t> more = dec.GenerateGreedy(out[0], (int)prompt.size(), n_new - 1);
        out.insert(out.end(), more.begin(), more.end());
      }
    }
    const auto t2 = clk::now();
    for (size_t i = 0; i < out.size(); i++) std::printf("%s%d", i ? " " : "", out[i]);
    std::printf("\n");
    const double tp = std::chrono::duration<double>(t1 - t0).count(), td = std::chrono::duration<double>(t2 - t1).count();
    std::printf("stats: prompt %zu tok %.1f tok/s, decode %d tok %.1f tok/s, cache %d\n", prompt.size(), prompt.size() / (tp > 0 ? tp : 1e-9),
                n_new - 1, (n_new - 1) / (td > 0 ? td : 1e-9), dec.SDPACacheLength());
  } catch (const caihip::CaiError& e) {
    std::fprintf(stderr, "caihip_run: error %d: %s\n", e.code, e.what());
    return 1;
  }
  return 0;
}
