// Self-checking exercise of the C++ host mirror (caihip_host.hpp); exits non-zero on the first failed check.
//   caihip_host_test MODEL.gguf
// Mirrors the calling sequences of the reference's tests: offload object upload -> compute -> finish
// (tests/TestNeuralNumerical.pas:66159-66164), cached decode == windowed forward, truncate / snapshot / restore
// (tests/TestNeuralFusedSDPA.pas:228-454, tests/TestNeuralDecode.pas:1708-1760).
#include "caihip_host.hpp"

#include <cmath>
#include <cstdlib>

static int g_failed = 0;
#define EXPECT(cond) do { if (!(cond)) { std::fprintf(stderr, "FAILED line %d: %s\n", __LINE__, #cond); g_failed++; } } while (0)

int main(int argc, char** argv)
{
  if (argc < 2) { std::fprintf(stderr, "usage: %s MODEL.gguf\n", argv[0]); return 2; }
  try {
    caihip::EnableHIP(0);
    {   // ---- offload object: per-row int8 weights, 2 input vectors, ReLU ----
      const int NumAs = 37, Size = 96, NumBs = 2;
      std::vector<int8_t> codes((size_t)NumAs * Size); std::vector<float> scales(NumAs), bias(NumAs), x((size_t)NumBs * Size);
      unsigned s = 12345u;
      auto rnd = [&]() { s = s * 1664525u + 1013904223u; return (int)((s >> 16) & 0xff) - 128; };
      for (auto& c : codes) { int v = rnd(); c = (int8_t)(v < -127 ? -127 : v); }
      for (int a = 0; a < NumAs; a++) { scales[a] = 0.001f * (float)(a + 1); bias[a] = 0.01f * (float)(a - 18); }
      for (auto& v : x) v = (float)rnd() / 64.0f;
      caihip::TDotProductSharedKernel k;
      int errors_seen = 0;
      k.ErrorProc = [&](const std::string&) { errors_seen++; };
      std::vector<float> y((size_t)NumAs * NumBs, -1.0f);
      EXPECT(k.ComputeInt8(x.data(), NumBs, 1) == CAI_ERR_STATE && errors_seen == 1);   // not prepared: logged, code returned, no throw
      EXPECT(!k.Int8Ready());
      EXPECT(k.PrepareForComputeInt8(codes.data(), scales.data(), NumAs, Size, bias.data()) == CAI_OK && k.Int8Ready());
      EXPECT(k.FinishAndLoadResult(y.data()) == CAI_ERR_STATE && errors_seen == 2);
      EXPECT(k.ComputeInt8(x.data(), NumBs, 1) == CAI_OK);
      EXPECT(k.FinishAndLoadResult(y.data()) == CAI_OK);
      double worst = 0.0;
      for (int b = 0; b < NumBs; b++)
        for (int a = 0; a < NumAs; a++) {
          double acc = 0.0;
          for (int i = 0; i < Size; i++) acc += (double)codes[(size_t)a * Size + i] * (double)x[(size_t)b * Size + i];
          double want = acc * scales[a] + bias[a]; if (want < 0) want = 0;     // y = act(scale * sum + bias)
          worst = std::fmax(worst, std::fabs(want - (double)y[(size_t)b * NumAs + a]));   // layout [b*NumAs + a]
        }
      EXPECT(worst < 1e-3);
      k.UnprepareForCompute();
      EXPECT(!k.Int8Ready());
    }
    {   // ---- session: windowed forward == token-at-a-time; truncate; snapshot / restore ----
      caihip::TNNetStreamingDecoder dec(argv[1], 32);
      const int32_t seq[] = {1, 5, 2, 7, 3, 0, 6, 4};
      const int n = 8;
      dec.Reset();
      std::vector<std::vector<float>> rows;
      for (int i = 0; i < n; i++) { dec.StepForward(&seq[i], 1, i); rows.push_back(dec.Output()); }
      EXPECT(dec.SDPACacheLength() == n);
      const int last_argmax = dec.ArgMaxRow();
      dec.Reset();
      EXPECT(dec.SDPACacheLength() == 0);
      dec.StepForward(seq, n, 0);                       // the whole window at once
      double worst = 0.0;
      for (size_t v = 0; v < rows[n - 1].size(); v++) worst = std::fmax(worst, std::fabs((double)rows[n - 1][v] - (double)dec.Output()[v]));
      EXPECT(worst < 1e-4 && dec.ArgMaxRow() == last_argmax && dec.SDPACacheLength() == n);
      // a window of up to eight tokens keeps EVERY row (the verify pass of speculative decoding)
      EXPECT(dec.WindowRows() == n);
      for (int r = 0; r < n; r++) {
        double w = 0.0;
        for (size_t v = 0; v < rows[(size_t)r].size(); v++) w = std::fmax(w, std::fabs((double)rows[(size_t)r][v] - (double)dec.OutputRow(r)[v]));
        EXPECT(w < 1e-4);
      }
      EXPECT((int)dec.HiddenState(n - 1).size() == dec.Config().d_model);
      // speculative rollback: drop 3 tokens, re-feed them, same logits
      dec.TruncateTo(5);
      EXPECT(dec.SDPACacheLength() == 5);
      for (int i = 5; i < n; i++) dec.StepForward(&seq[i], 1, i);
      worst = 0.0;
      for (size_t v = 0; v < rows[n - 1].size(); v++) worst = std::fmax(worst, std::fabs((double)rows[n - 1][v] - (double)dec.Output()[v]));
      EXPECT(worst < 1e-5);
      // prefix reuse: snapshot after 4 tokens, run on, restore, continue: identical to the first pass
      dec.Reset();
      dec.StepForward(seq, 4, 0);
      caihip::TNNetDecoderSessionSnapshot* snap = dec.Snapshot();
      for (int i = 4; i < n; i++) dec.StepForward(&seq[i], 1, i);
      dec.RestoreSnapshot(snap);
      EXPECT(dec.SDPACacheLength() == 4);
      dec.StepForward(&seq[4], 1, 4);
      worst = 0.0;
      for (size_t v = 0; v < rows[4].size(); v++) worst = std::fmax(worst, std::fabs((double)rows[4][v] - (double)dec.Output()[v]));
      EXPECT(worst < 1e-5);
      delete snap;
      // greedy chain on the device == stepping from the host
      dec.Reset();
      dec.StepForward(seq, 4, 0);
      const int32_t first = dec.ArgMaxRow();
      std::vector<int32_t> host_chain; int32_t t = first;
      for (int k = 0; k < 6; k++) { dec.StepForward(&t, 1, 4 + k); t = dec.ArgMaxRow(); host_chain.push_back(t); }
      dec.TruncateTo(4);
      EXPECT(dec.GenerateGreedy(first, 4, 6) == host_chain);
      // prompt-lookup generation writes the same tokens, in at most as many passes
      dec.TruncateTo(4);
      { int passes = 0; std::vector<int32_t> ctx(seq, seq + 4); ctx.push_back(first);
        EXPECT(dec.GenerateLookup(ctx, 1, 4, 6, &passes) == host_chain && passes >= 1 && passes <= 6); }
      // sampled decode: the candidate prefix of the resident row is the sorted soft-max head, and the samplers draw from it
      {
        dec.Reset();
        dec.StepForward(seq, 4, 0);
        const std::vector<float>& lg = dec.Output();
        caihip::TNNetCandidates c = dec.Candidates(8);
        EXPECT(c.Count() == 8 && c.Token[0] == dec.ArgMaxRow());
        double mx = lg[0]; for (float v : lg) mx = std::fmax(mx, (double)v);
        double sum = 0; for (float v : lg) sum += std::exp((double)v - mx);
        for (int i = 0; i < c.Count(); i++) {
          EXPECT(std::fabs(std::exp((double)lg[(size_t)c.Token[(size_t)i]] - mx) / sum - (double)c.Score[(size_t)i]) < 1e-5);
          if (i) EXPECT(c.Score[(size_t)i] <= c.Score[(size_t)i - 1]);
        }
        EXPECT(caihip::SampleTopK(c, 4, 0.0) == c.Token[0] && caihip::SampleTopK(c, 4, 0.99) == c.Token[3]);
        EXPECT(caihip::SampleWeightedTopK(c, 8, 0.0) == c.Token[0]);
        EXPECT(caihip::SampleTopP(c, 2.0f, 0.5) == -1);                    // the prefix cannot hold more than all the mass
        EXPECT(caihip::SampleTopP(c, c.Score[0] * 0.5f, 0.7) == c.Token[0]); // the first token alone exceeds P: fallback to it
        EXPECT(caihip::SampleMinP(c, 0.999f, 0.3) == c.Token[0] || c.Score[1] >= 0.999f * c.Score[0]);
        caihip::TNNetTokenHistory hist;
        for (int i = 0; i < 4; i++) hist.RegisterToken(seq[i]);
        hist.RegisterToken(c.Token[0]); hist.RegisterToken(c.Token[0]);
        caihip::TNNetCandidates pen = dec.Candidates(8, 1.0f, &hist, 1.5f, 0.5f, 0.5f);
        float before = c.Score[0], after = 0;
        for (int i = 0; i < pen.Count(); i++) if (pen.Token[(size_t)i] == c.Token[0]) after = pen.Score[(size_t)i];
        EXPECT(after < before);                                            // a repeated token loses mass
        caihip::TNNetCandidates cold = dec.Candidates(2, 1e-9f);
        EXPECT(cold.Token[0] == dec.ArgMaxRow() && cold.Score[0] > 0.999f); // T -> 0 is greedy
      }
      // streaming past the cache with sink + recent-window eviction (tests/TestNeuralDecode.pas:3930-3975)
      {
        dec.Reset();
        dec.EnableEviction(2, 6);
        for (int i = 0; i < 40; i++) {
          dec.StepForward(&seq[i % n], 1, i);
          EXPECT(dec.SDPACacheLength() == (i + 1 <= 8 ? i + 1 : 8));
        }
        bool refused = false;
        try { dec.DisableEviction(); } catch (const caihip::CaiError&) { refused = true; }
        EXPECT(refused);                                                   // past the cap the middle is gone
        dec.Reset();
        dec.DisableEviction();
        bool refused2 = false;
        dec.StepForward(seq, 2, 0);
        try { dec.EnableInt8KVCache(); } catch (const caihip::CaiError&) { refused2 = true; }
        EXPECT(refused2);                                                  // only a fresh session switches storage
        dec.Reset();
        dec.EnableInt8KVCache();
        dec.StepForward(seq, n, 0);
        double drift = 0.0;
        for (size_t v = 0; v < rows[n - 1].size(); v++) drift = std::fmax(drift, std::fabs((double)rows[n - 1][v] - (double)dec.Output()[v]));
        EXPECT(drift < 0.1 && dec.SDPACacheLength() == n);
        dec.Reset();
        dec.DisableInt8KVCache();
      }
      // importer errors raise
      bool raised = false;
      try { caihip::TNNetStreamingDecoder bad("/nonexistent/model.gguf"); } catch (const caihip::CaiError& e) { raised = e.code != CAI_OK; }
      EXPECT(raised);
    }
  } catch (const caihip::CaiError& e) {
    std::fprintf(stderr, "caihip_host_test: error %d: %s\n", e.code, e.what());
    return 1;
  }
  if (g_failed) { std::fprintf(stderr, "%d check(s) failed\n", g_failed); return 1; }
  std::printf("host mirror ok\n");
  return 0;
}
