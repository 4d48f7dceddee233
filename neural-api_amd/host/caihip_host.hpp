// C++ host-side mirror of the two reference objects that sit on the decode path, written over the C ABI of
// include/caihip.h (this is the executable twin of the Free Pascal adapter described for maintainers; the
// reference's own host language has no compiler in this build image):
//
//   TDotProductSharedKernel  (neural/neuralopencl.pas:245-388, 844-1104): per-layer offload object.
//       PrepareForComputeInt8 -> blocking one-time upload of the weights; ComputeInt8 -> enqueue one product;
//       FinishAndLoadResult -> block and write NumAs*NumBs floats laid out [b*NumAs + a].
//       Errors are reported through ErrorProc and the call returns a code; nothing is thrown (957-969).
//   TNNetStreamingDecoder    (neural/neuraldecode.pas:1210-1333, 5696-5843): session over a whole decoder.
//       Reset, StepForward(window, AbsPos), TruncateTo, Snapshot / RestoreSnapshot, EnableEviction / DisableEviction,
//       SDPACacheLength, Output.
//       Importer-level failures raise (EPretrainedImportError / EGGUFError in the reference): here CaiError.
#pragma once
#include <caihip.h>

#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <functional>
#include <stdexcept>
#include <string>
#include <vector>

namespace caihip {

inline std::string LastError()
{
  char buf[1024];
  cai_last_error(buf, (int)sizeof buf);
  return std::string(buf);
}

struct CaiError : std::runtime_error {
  int code;
  CaiError(int c, const std::string& m) : std::runtime_error(m), code(c) {}
};
inline void Check(int rc) { if (rc != CAI_OK) throw CaiError(rc, LastError()); }

// EnableOpenCL analogue (neural/neuralchatengine.pas:1156-1157): arm the device once per process.
inline void EnableHIP(int device = 0) { Check(cai_init(device)); }

class TDotProductSharedKernel {
 public:
  std::function<void(const std::string&)> ErrorProc = [](const std::string& m) { std::fprintf(stderr, "%s\n", m.c_str()); };

  ~TDotProductSharedKernel() { UnprepareForCompute(); }

  // per-row symmetric int8 codes + fp32 row scales (the reference's own resident format)
  int PrepareForComputeInt8(const int8_t* pCodes, const float* pScales, int NumAs, int pSize, const float* pBias = nullptr)
  {
    UnprepareForCompute();
    return Report(cai_qw_create_int8row(NumAs, pSize, pCodes, pScales, pBias, &w_), NumAs, pSize);
  }
  // GGUF blocks in stored order (CAI_Q8_0 / CAI_Q4_0 / CAI_Q4_K / CAI_F16 / CAI_F32): no dequantised copy is ever made
  int PrepareForComputeBlocks(int qtype, const void* pBlocks, int NumAs, int pSize, const float* pBias = nullptr)
  {
    UnprepareForCompute();
    return Report(cai_qw_create(qtype, NumAs, pSize, pBlocks, pBias, &w_), NumAs, pSize);
  }
  bool Int8Ready() const { return w_ != nullptr; }

  // VBs: NumBs input vectors of pSize floats.  ActFN: 0 none, 1 ReLU, 2 sigmoid, 3 tanh (neural/neural.cl:114-146);
  // bias is added before the activation.
  int ComputeInt8(const float* VBs, int NumBs, int ActFN = 0)
  {
    if (!w_) return Fail(CAI_ERR_STATE, "ComputeInt8 before PrepareForComputeInt8");
    result_.assign((size_t)NumBs * (size_t)num_as_, 0.0f);
    const int rc = cai_qgemv(w_, VBs, NumBs, result_.data(), ActFN, 0);
    if (rc) return Fail(rc, LastError());
    pending_ = true;
    return CAI_OK;
  }
  int FinishAndLoadResult(float* Results)
  {
    if (!pending_) return Fail(CAI_ERR_STATE, "FinishAndLoadResult without a ComputeInt8 in flight");
    for (size_t i = 0; i < result_.size(); i++) Results[i] = result_[i];
    pending_ = false;
    return CAI_OK;
  }
  void UnprepareForCompute() { if (w_) { cai_qw_destroy(w_); w_ = nullptr; } pending_ = false; }

 private:
  int Report(int rc, int NumAs, int pSize) { if (rc) return Fail(rc, LastError()); num_as_ = NumAs; size_ = pSize; return CAI_OK; }
  int Fail(int rc, const std::string& m) { if (ErrorProc) ErrorProc(m); return rc; }
  cai_qw_t w_ = nullptr;
  int num_as_ = 0, size_ = 0;
  bool pending_ = false;
  std::vector<float> result_;
};

class TNNetDecoderSessionSnapshot {
 public:
  explicit TNNetDecoderSessionSnapshot(cai_kv_snap_t s) : s_(s) {}
  ~TNNetDecoderSessionSnapshot() { if (s_) cai_kv_snap_destroy(s_); }
  TNNetDecoderSessionSnapshot(const TNNetDecoderSessionSnapshot&) = delete;
  TNNetDecoderSessionSnapshot& operator=(const TNNetDecoderSessionSnapshot&) = delete;
  cai_kv_snap_t handle() const { return s_; }
 private:
  cai_kv_snap_t s_;
};

// The candidate prefix the device hands back (descending probabilities) and the reference's samplers over it.  The
// draws are the HOST's: u in [0,1) stands where the reference calls Random, so a host keeps its own generator and seed.
struct TNNetCandidates {
  std::vector<int32_t> Token;
  std::vector<float> Score;
  int Count() const { return (int)Token.size(); }
};

// TNNetSamplerTopK (neural/neuralvolume.pas:4716-4731): uniform over the K most probable.
inline int32_t SampleTopK(const TNNetCandidates& c, int TopK, double u)
{
  int n = std::min(std::max(TopK, 1), c.Count());
  if (n <= 0) return 0;
  return c.Token[(size_t)std::min(n - 1, (int)(u * n))];
}
// TNNetSamplerWeightedTopK (4749-4786): proportional to the kept probabilities; TopK <= 0 keeps the whole prefix.
inline int32_t SampleWeightedTopK(const TNNetCandidates& c, int TopK, double u)
{
  if (c.Count() == 0) return 0;
  int kept = TopK; if (kept <= 0 || kept > c.Count()) kept = c.Count();
  float sum = 0; for (int i = 0; i < kept; i++) sum += c.Score[(size_t)i];
  if (sum <= 0) return c.Token[0];
  const float roll = (float)u * sum; float cum = 0;
  for (int i = 0; i < kept; i++) { cum += c.Score[(size_t)i]; if (roll < cum) return c.Token[(size_t)i]; }
  return c.Token[(size_t)kept - 1];
}
// TNNetSamplerTopP (4548-4600): the first index whose cumulative mass exceeds TopP bounds a window that is drawn from
// UNIFORMLY.  Returns -1 when the prefix does not hold TopP of the mass: ask for a wider prefix (the reference re-sorts
// the whole row in that case) or fall back to the logits row.
inline int32_t SampleTopP(const TNNetCandidates& c, float TopP, double u)
{
  if (c.Count() == 0) return 0;
  float cum = 0; int threshold = -1;
  for (int i = 0; i < c.Count(); i++) { cum += c.Score[(size_t)i]; if (cum > TopP) { threshold = i; break; } }
  if (threshold < 0) return -1;
  if (threshold == 0) return c.Token[0];
  return c.Token[(size_t)std::min(threshold - 1, (int)(u * threshold))];
}
// TNNetSamplerMinP (4621-4665): keep p >= MinP * max p, weighted draw.  Returns -1 when the whole prefix passes the cut
// (the kept set may reach beyond it).
inline int32_t SampleMinP(const TNNetCandidates& c, float MinP, double u, bool PrefixIsWholeRow = false)
{
  if (c.Count() == 0) return 0;
  const float cut = MinP * c.Score[0];
  int kept = 0; float sum = 0;
  for (int i = 0; i < c.Count(); i++) { if (c.Score[(size_t)i] >= cut) { kept++; sum += c.Score[(size_t)i]; } else break; }
  if (kept == c.Count() && !PrefixIsWholeRow) return -1;
  if (kept == 0 || sum <= 0) return c.Token[0];
  const float roll = (float)u * sum; float cum = 0;
  for (int i = 0; i < kept; i++) { cum += c.Score[(size_t)i]; if (roll < cum) return c.Token[(size_t)i]; }
  return c.Token[(size_t)kept - 1];
}

// TNNetTokenHistoryPenalty's bookkeeping (neural/neuralvolume.pas:5266-5292): distinct ids + occurrence counts.
class TNNetTokenHistory {
 public:
  void RegisterToken(int32_t TokenId)
  {
    if (TokenId < 0) return;
    for (size_t i = 0; i < ids_.size(); i++) if (ids_[i] == TokenId) { counts_[i]++; return; }
    ids_.push_back(TokenId); counts_.push_back(1);
  }
  void ResetHistory() { ids_.clear(); counts_.clear(); }
  const std::vector<int32_t>& Ids() const { return ids_; }
  const std::vector<int32_t>& Counts() const { return counts_; }
 private:
  std::vector<int32_t> ids_, counts_;
};

class TNNetStreamingDecoder {
 public:
  // BuildLlamaFromGGUF + TNNetStreamingDecoder.Create(pNet, pMaxCacheLen): pMaxCacheLen <= 0 takes the file's context length
  TNNetStreamingDecoder(const std::string& GGUFFileName, int pMaxCacheLen = 0, bool pF16KV = false)
  {
    Check(cai_decoder_load_gguf(GGUFFileName.c_str(), pMaxCacheLen, 1, pF16KV ? CAI_KV_F16 : CAI_KV_F32, &d_));
    Check(cai_decoder_get_config(d_, &cfg_));
    logits_.resize((size_t)cfg_.vocab);
  }
  ~TNNetStreamingDecoder() { if (d_) cai_decoder_destroy(d_); }
  TNNetStreamingDecoder(const TNNetStreamingDecoder&) = delete;
  TNNetStreamingDecoder& operator=(const TNNetStreamingDecoder&) = delete;

  const cai_decoder_config& Config() const { return cfg_; }
  void Reset() { Check(cai_decoder_reset(d_, 0)); }
  // One streamed forward of a window of token ids; AbsPos is the absolute position of the FIRST token of the window.
  // After it, Output() holds the logits of the window's last token and ArgMaxRow() their arg-max (lowest index on ties).
  // A window of 2..8 tokens (the verify pass of speculative decoding, neural/neuraldecode.pas:1151-1183) also keeps every
  // row: OutputRow(r) / ArgMaxRows()[r] belong to position AbsPos + r.  Longer windows are prompt passes (last row only).
  void StepForward(const int32_t* Tokens, int Count, int AbsPos)
  {
    rows_ = 0;
    if (Count == 1) { int32_t p = AbsPos; Check(cai_decoder_step(d_, Tokens, &p, 1, logits_.data(), &argmax_)); }
    else if (Count <= 8) {
      window_.resize((size_t)Count * (size_t)cfg_.vocab); argmax_rows_.resize((size_t)Count);
      Check(cai_decoder_step_window(d_, 0, Tokens, Count, AbsPos, window_.data(), argmax_rows_.data()));
      rows_ = Count;
      std::copy(window_.end() - cfg_.vocab, window_.end(), logits_.begin());
      argmax_ = argmax_rows_.back();
    }
    else Check(cai_decoder_prefill(d_, 0, Tokens, Count, AbsPos, logits_.data(), &argmax_));
  }
  int WindowRows() const { return rows_; }
  const float* OutputRow(int r) const { return window_.data() + (size_t)r * (size_t)cfg_.vocab; }
  const std::vector<int32_t>& ArgMaxRows() const { return argmax_rows_; }
  // HiddenState (neural/neuraldecode.pas:1314-1321): the input of the vocabulary projection for a row of the last step or window
  std::vector<float> HiddenState(int Row = 0)
  {
    std::vector<float> h((size_t)cfg_.d_model);
    Check(cai_decoder_hidden_state(d_, Row, h.data()));
    return h;
  }
  // DecodePromptLookup on the cached session (neural/neuraldecode.pas:7767-7866): Context minus its last token must be in
  // the cache; returns n greedy tokens, *Passes the number of window steps taken
  std::vector<int32_t> GenerateLookup(const std::vector<int32_t>& Context, int MatchLen, int NumDraft, int n, int* Passes = nullptr)
  {
    std::vector<int32_t> out((size_t)n); int32_t passes = 0;
    Check(cai_decoder_generate_lookup(d_, Context.data(), (int)Context.size(), MatchLen, NumDraft, n, out.data(), &passes));
    if (Passes) *Passes = passes;
    return out;
  }
  void TruncateTo(int CommittedLen) { Check(cai_decoder_truncate(d_, 0, CommittedLen)); }
  int SDPACacheLength(int Index = 0) const { int n = 0; Check(cai_decoder_cache_rows(d_, 0, Index, &n)); return n; }
  // neural/neuraldecode.pas:5722-5735
  void EnableEviction(int SinkTokens, int RecentWindow) { Check(cai_decoder_set_eviction(d_, SinkTokens, RecentWindow)); }
  void DisableEviction() { Check(cai_decoder_set_eviction(d_, 0, 0)); }
  // neural/neuraldecode.pas:1277-1290: only on a fresh session
  void EnableInt8KVCache() { Check(cai_decoder_set_kv_dtype(d_, CAI_KV_I8)); }
  void DisableInt8KVCache() { Check(cai_decoder_set_kv_dtype(d_, CAI_KV_F32)); }
  TNNetDecoderSessionSnapshot* Snapshot() { cai_kv_snap_t s = nullptr; Check(cai_decoder_snapshot(d_, 0, &s)); return new TNNetDecoderSessionSnapshot(s); }
  void RestoreSnapshot(const TNNetDecoderSessionSnapshot* Snap) { Check(cai_decoder_restore(d_, 0, Snap->handle())); }
  const std::vector<float>& Output() const { return logits_; }
  int ArgMaxRow() const { return argmax_; }
  // RowSoftMax -> penalty -> temperature on the device, over the (last) row of the last StepForward; the m most probable
  // tokens come back instead of the row (neural/neuralchatengine.pas:1495-1501)
  TNNetCandidates Candidates(int m, float Temperature = 1.0f, const TNNetTokenHistory* History = nullptr,
                             float RepetitionPenalty = 1.0f, float FrequencyPenalty = 0.0f, float PresencePenalty = 0.0f)
  {
    TNNetCandidates c; c.Token.resize((size_t)m); c.Score.resize((size_t)m);
    int n = 0;
    Check(cai_decoder_candidates(d_, rows_ ? rows_ - 1 : 0, History ? History->Ids().data() : nullptr, History ? History->Counts().data() : nullptr,
                                 History ? (int)History->Ids().size() : 0, RepetitionPenalty, FrequencyPenalty, PresencePenalty,
                                 Temperature, m, c.Token.data(), c.Score.data(), &n));
    c.Token.resize((size_t)n); c.Score.resize((size_t)n);
    return c;
  }
  // Greedy fast path of the chat engine (neural/neuralchatengine.pas:1493-1494): n tokens chained on the device.
  std::vector<int32_t> GenerateGreedy(int32_t FirstToken, int AbsPos, int n)
  {
    std::vector<int32_t> out((size_t)n);
    Check(cai_decoder_generate(d_, FirstToken, AbsPos, n, out.data()));
    return out;
  }

 private:
  cai_decoder_t d_ = nullptr;
  cai_decoder_config cfg_{};
  std::vector<float> logits_, window_;
  std::vector<int32_t> argmax_rows_;
  int rows_ = 0;
  int32_t argmax_ = -1;
};

}  // namespace caihip
