// Library lifetime, error reporting, device buffers and resident weight matrices.
#include "cai_internal.hpp"

#include <stdarg.h>
#include <string.h>
#include <mutex>
#include <algorithm>

namespace cai {

static Context g_ctx;
static std::recursive_mutex g_api_mu;            // entry points call one another (generate -> step), hence recursive
static thread_local std::string t_err;           // the message belongs to the thread whose call failed
static thread_local int t_device = -1;           // HIP's current device is a per-thread setting

Context& ctx() { return g_ctx; }

// One call into the library at a time: the context's stream, staging buffers and scratch are shared by every handle, and
// all device work is ordered on the one stream anyway.  A thread that enters for the first time (or after cai_init chose
// another device) makes the library's device its current one.
ApiLock::ApiLock()
{
  g_api_mu.lock();
  if (g_ctx.ready && t_device != g_ctx.device) { (void)hipSetDevice(g_ctx.device); t_device = g_ctx.device; }
}
ApiLock::~ApiLock() { g_api_mu.unlock(); }

int set_error(int code, const char* fmt, ...)
{
  char buf[512];
  va_list ap; va_start(ap, fmt); vsnprintf(buf, sizeof(buf), fmt, ap); va_end(ap);
  t_err = buf;
  return code;
}

int hip_fail(hipError_t e, const char* what, const char* file, int line)
{
  (void)hipGetLastError();   // the runtime keeps the error until someone reads it: a later, unrelated launch check would report it again
  return set_error(e == hipErrorOutOfMemory ? CAI_ERR_NOMEM : CAI_ERR_HIP, "%s failed: %s (%s:%d)", what, hipGetErrorString(e), file, line);
}

unsigned long long* timeline_next(int n_wg)
{
  Context::Timeline& t = g_ctx.tl;
  if (!t.armed || t.used + (size_t)n_wg * TL_STAMPS > t.cap) return nullptr;
  unsigned long long* r = t.buf + t.used;
  t.launches.push_back(t.cls); t.launches.push_back(n_wg); t.launches.push_back((int32_t)t.used);
  t.used += (size_t)n_wg * TL_STAMPS;
  return r;
}

int ensure_stage(void** p, size_t* cap, size_t need)
{
  if (*cap >= need) return CAI_OK;
  CAI_HIP(hipStreamSynchronize(g_ctx.stream));
  if (*p) { (void)hipFree(*p); *p = nullptr; *cap = 0; }
  size_t want = need < (1u << 20) ? (1u << 20) : need;
  CAI_HIP(hipMalloc(p, want));
  *cap = want;
  return CAI_OK;
}

int64_t block_elems(int qt)
{
  switch (qt) { case CAI_F32: case CAI_F16: case CAI_I8ROW: return 1; case CAI_Q4_0: case CAI_Q8_0: return 32; case CAI_Q4_K: case CAI_Q6_K: return 256; }
  if (raw_block_type(qt)) return raw_block_elems(qt);
  return -1;
}
int64_t block_bytes(int qt)
{
  switch (qt) { case CAI_F32: return 4; case CAI_F16: return 2; case CAI_I8ROW: return 1; case CAI_Q4_0: return 18; case CAI_Q8_0: return 34; case CAI_Q4_K: return 144; case CAI_Q6_K: return 210; }
  if (raw_block_type(qt)) return raw_block_bytes(qt);
  return -1;
}

}  // namespace cai

using namespace cai;

extern "C" int cai_init(int device_ordinal)
{
  CAI_ENTER();
  Context& c = ctx();
  if (c.ready) {
    if (c.device == device_ordinal) return CAI_OK;
    return set_error(CAI_ERR_STATE, "cai_init: already initialised on device %d", c.device);
  }
  int n = 0;
  CAI_HIP(hipGetDeviceCount(&n));
  if (device_ordinal < 0 || device_ordinal >= n) return set_error(CAI_ERR_INVALID, "cai_init: device %d of %d", device_ordinal, n);
  CAI_HIP(hipSetDevice(device_ordinal));
  hipDeviceProp_t prop;
  CAI_HIP(hipGetDeviceProperties(&prop, device_ordinal));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return set_error(CAI_ERR_UNSUPPORTED, "cai_init: device %d is %s; this library is built for gfx950 only", device_ordinal, prop.gcnArchName);
  snprintf(c.name, sizeof(c.name), "%s (%s, %d CUs)", prop.name, prop.gcnArchName, prop.multiProcessorCount);
  c.n_cu = prop.multiProcessorCount;
  c.device = device_ordinal;
  CAI_HIP(hipStreamCreateWithFlags(&c.stream, hipStreamNonBlocking));
  CAI_HIP(hipEventCreate(&c.ev0));
  CAI_HIP(hipEventCreate(&c.ev1));
  CAI_HIP(hipMalloc(&c.d_small, 1024 * sizeof(int32_t)));
  CAI_HIP(hipHostMalloc(&c.h_small, 1024 * sizeof(int32_t), hipHostMallocDefault));
  { const int rc = noalloc_setup(device_ordinal); if (rc) return rc; }
  c.ready = true;
  return CAI_OK;
}

extern "C" int cai_shutdown(void)
{
  CAI_ENTER();
  Context& c = ctx();
  if (!c.ready) return CAI_OK;
  (void)hipStreamSynchronize(c.stream);
  if (c.stage_in) (void)hipFree(c.stage_in);
  if (c.stage_out) (void)hipFree(c.stage_out);
  if (c.stage_sample) (void)hipFree(c.stage_sample);
  nb_release(); ra_release(); prefill_release();
  if (c.d_small) (void)hipFree(c.d_small);
  if (c.h_small) (void)hipHostFree(c.h_small);
  if (c.tl.buf) (void)hipFree(c.tl.buf);
  (void)hipEventDestroy(c.ev0); (void)hipEventDestroy(c.ev1);
  (void)hipStreamDestroy(c.stream);
  c = Context();
  return CAI_OK;
}

extern "C" int cai_last_error(char* buf, int buf_len)
{
  if (!buf || buf_len <= 0) return CAI_ERR_INVALID;
  snprintf(buf, (size_t)buf_len, "%s", t_err.c_str());
  return CAI_OK;
}

extern "C" int cai_device_name(char* buf, int buf_len)
{
  CAI_ENTER();
  CAI_READY();
  if (!buf || buf_len <= 0) return CAI_ERR_INVALID;
  snprintf(buf, (size_t)buf_len, "%s", ctx().name);
  return CAI_OK;
}

extern "C" int cai_sync(void) { CAI_ENTER(); CAI_READY(); CAI_HIP(hipStreamSynchronize(ctx().stream)); return CAI_OK; }
extern "C" int cai_get_stream(void** s) { CAI_ENTER(); CAI_READY(); CAI_REQUIRE(s, "cai_get_stream: null out"); *s = (void*)ctx().stream; return CAI_OK; }
extern "C" int cai_timer_start(void) { CAI_ENTER(); CAI_READY(); CAI_HIP(hipEventRecord(ctx().ev0, ctx().stream)); return CAI_OK; }
extern "C" int cai_timer_stop(float* ms)
{
  CAI_ENTER();
  CAI_READY(); CAI_REQUIRE(ms, "cai_timer_stop: null out");
  CAI_HIP(hipEventRecord(ctx().ev1, ctx().stream));
  CAI_HIP(hipEventSynchronize(ctx().ev1));
  CAI_HIP(hipEventElapsedTime(ms, ctx().ev0, ctx().ev1));
  return CAI_OK;
}

extern "C" int cai_dev_alloc(int64_t bytes, void** out)
{
  CAI_ENTER();
  CAI_READY(); CAI_REQUIRE(out && bytes > 0, "cai_dev_alloc: bad argument");
  CAI_HIP(hipMalloc(out, (size_t)bytes));
  return CAI_OK;
}
extern "C" int cai_dev_free(void* p) { CAI_ENTER(); CAI_READY(); if (p) { CAI_HIP(hipStreamSynchronize(ctx().stream)); CAI_HIP(hipFree(p)); } return CAI_OK; }
extern "C" int cai_dev_upload(void* d, const void* h, int64_t bytes)
{
  CAI_ENTER();
  CAI_READY(); CAI_REQUIRE(d && h && bytes >= 0, "cai_dev_upload: bad argument");
  CAI_HIP(hipMemcpyAsync(d, h, (size_t)bytes, hipMemcpyHostToDevice, ctx().stream));
  CAI_HIP(hipStreamSynchronize(ctx().stream));
  return CAI_OK;
}
extern "C" int cai_dev_download(void* h, const void* d, int64_t bytes)
{
  CAI_ENTER();
  CAI_READY(); CAI_REQUIRE(d && h && bytes >= 0, "cai_dev_download: bad argument");
  CAI_HIP(hipMemcpyAsync(h, d, (size_t)bytes, hipMemcpyDeviceToHost, ctx().stream));
  CAI_HIP(hipStreamSynchronize(ctx().stream));
  return CAI_OK;
}

namespace cai {
__global__ __launch_bounds__(256) void copy16_kernel(const uint4* src, uint4* dst, size_t n16)
{
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; const size_t stride = (size_t)gridDim.x * 256;
  for (; i < n16; i += stride) dst[i] = src[i];
}
}  // namespace cai

extern "C" int cai_dev_copy(void* dst, const void* src, int64_t bytes)
{
  CAI_ENTER();
  CAI_READY(); CAI_REQUIRE(dst && src && bytes > 0 && bytes % 16 == 0, "cai_dev_copy: bad argument");
  const size_t n16 = (size_t)bytes / 16;
  const int grid = (int)std::min<size_t>((n16 + 255) / 256, 8192);
  hipLaunchKernelGGL(cai::copy16_kernel, dim3(grid), dim3(256), 0, ctx().stream, (const uint4*)src, (uint4*)dst, n16);
  CAI_HIP(hipGetLastError());
  return CAI_OK;
}

// ------------------------------------------------------------------------------------------
// resident weights
// ------------------------------------------------------------------------------------------
static void qw_free(cai_qw_s* w)
{
  if (w->data) (void)hipFree(w->data);
  if (w->aux) (void)hipFree(w->aux);
  if (w->bias) (void)hipFree(w->bias);
  delete w;
}

static int qw_set_bias(cai_qw_s* w, const float* bias)
{
  if (!bias) return CAI_OK;
  CAI_HIP(hipMalloc(&w->bias, (size_t)w->rows * 4));
  CAI_HIP(hipMemcpyAsync(w->bias, bias, (size_t)w->rows * 4, hipMemcpyHostToDevice, ctx().stream));
  w->algo_bytes += w->rows * 4;
  return CAI_OK;
}

extern "C" int cai_qw_create(int qtype, int64_t rows, int64_t cols, const void* blocks, const float* bias, cai_qw_t* out)
{
  CAI_ENTER();
  CAI_READY();
  CAI_REQUIRE(out && blocks, "cai_qw_create: null argument");
  CAI_REQUIRE(rows > 0 && cols > 0 && rows < (1ll << 31) && cols < (1ll << 31), "cai_qw_create: bad shape %lld x %lld", (long long)rows, (long long)cols);
  const int64_t be = block_elems(qtype);
  if (be < 0 || qtype == CAI_I8ROW) return set_error(CAI_ERR_UNSUPPORTED, "cai_qw_create: unsupported weight type %d", qtype);
  // a quant block never straddles a row (neural/neuralgguf.pas:226-236, 1165-1187)
  CAI_REQUIRE(cols % be == 0, "cai_qw_create: %lld columns is not a whole number of %lld-element blocks", (long long)cols, (long long)be);
  Context& c = ctx();
  cai_qw_s* w = new cai_qw_s();
  w->qtype = qtype; w->rows = rows; w->cols = cols;
  const int64_t raw_bytes = rows * (cols / be) * block_bytes(qtype);
  w->algo_bytes = raw_bytes;
  int rc = CAI_OK;
  auto fail = [&](int code) { qw_free(w); return code; };
  if (qtype == CAI_Q8_0 || qtype == CAI_Q4_0) {
    const int64_t n_blocks = rows * (cols / 32);
    const int bb = (int)block_bytes(qtype);
    w->data_bytes = n_blocks * (bb - 2); w->aux_bytes = n_blocks * 2;
    void* raw = nullptr;
    if (hipMalloc(&raw, (size_t)raw_bytes) != hipSuccess) return (void)hipGetLastError(), fail(set_error(CAI_ERR_NOMEM, "cai_qw_create: out of device memory (%lld bytes staging)", (long long)raw_bytes));
    hipError_t e = hipMalloc((void**)&w->data, (size_t)w->data_bytes);
    if (e == hipSuccess) e = hipMalloc((void**)&w->aux, (size_t)w->aux_bytes);
    if (e == hipSuccess) e = hipMemcpyAsync(raw, blocks, (size_t)raw_bytes, hipMemcpyDefault, c.stream);
    if (e == hipSuccess) { launch_split_blocks((const uint8_t*)raw, bb, n_blocks, w->data, (uint16_t*)w->aux); e = hipStreamSynchronize(c.stream); }
    (void)hipFree(raw);
    if (e != hipSuccess) return fail(hip_fail(e, "cai_qw_create upload", __FILE__, __LINE__));
  } else if (qtype == CAI_Q6_K) {
    const int64_t n_blocks = rows * (cols / 256);
    w->data_bytes = n_blocks * 192; w->aux_bytes = n_blocks * 18;
    void* raw = nullptr;
    if (hipMalloc(&raw, (size_t)raw_bytes) != hipSuccess) return (void)hipGetLastError(), fail(set_error(CAI_ERR_NOMEM, "cai_qw_create: out of device memory (%lld bytes staging)", (long long)raw_bytes));
    hipError_t e = hipMalloc((void**)&w->data, (size_t)w->data_bytes);
    if (e == hipSuccess) e = hipMalloc((void**)&w->aux, (size_t)w->aux_bytes);
    if (e == hipSuccess) e = hipMemcpyAsync(raw, blocks, (size_t)raw_bytes, hipMemcpyDefault, c.stream);
    if (e == hipSuccess) { launch_split_q6k((const uint8_t*)raw, n_blocks, w->data, w->aux, (uint16_t*)(w->aux + n_blocks * 16)); e = hipStreamSynchronize(c.stream); }
    (void)hipFree(raw);
    if (e != hipSuccess) return fail(hip_fail(e, "cai_qw_create upload", __FILE__, __LINE__));
  } else {
    w->data_bytes = raw_bytes;
    hipError_t e = hipMalloc((void**)&w->data, (size_t)raw_bytes);
    if (e == hipSuccess) e = hipMemcpyAsync(w->data, blocks, (size_t)raw_bytes, hipMemcpyDefault, c.stream);
    if (e != hipSuccess) return fail(hip_fail(e, "cai_qw_create upload", __FILE__, __LINE__));
  }
  if ((rc = qw_set_bias(w, bias))) return fail(rc);
  if (hipStreamSynchronize(c.stream) != hipSuccess) return fail(set_error(CAI_ERR_HIP, "cai_qw_create: stream sync failed"));
  *out = w;
  return CAI_OK;
}

extern "C" int cai_qw_create_int8row(int64_t rows, int64_t cols, const int8_t* codes, const float* scales, const float* bias, cai_qw_t* out)
{
  CAI_ENTER();
  CAI_READY();
  CAI_REQUIRE(out && codes && scales, "cai_qw_create_int8row: null argument");
  CAI_REQUIRE(rows > 0 && cols > 0 && rows < (1ll << 31) && cols < (1ll << 31), "cai_qw_create_int8row: bad shape");
  Context& c = ctx();
  cai_qw_s* w = new cai_qw_s();
  w->qtype = CAI_I8ROW; w->rows = rows; w->cols = cols;
  w->data_bytes = rows * cols; w->aux_bytes = rows * 4; w->algo_bytes = w->data_bytes + w->aux_bytes;
  hipError_t e = hipMalloc((void**)&w->data, (size_t)w->data_bytes);
  if (e == hipSuccess) e = hipMalloc((void**)&w->aux, (size_t)w->aux_bytes);
  if (e == hipSuccess) e = hipMemcpyAsync(w->data, codes, (size_t)w->data_bytes, hipMemcpyDefault, c.stream);
  if (e == hipSuccess) e = hipMemcpyAsync(w->aux, scales, (size_t)w->aux_bytes, hipMemcpyDefault, c.stream);
  if (e != hipSuccess) { qw_free(w); return hip_fail(e, "cai_qw_create_int8row upload", __FILE__, __LINE__); }
  const int rc = qw_set_bias(w, bias);
  if (rc) { qw_free(w); return rc; }
  if (hipStreamSynchronize(c.stream) != hipSuccess) { qw_free(w); return set_error(CAI_ERR_HIP, "cai_qw_create_int8row: stream sync failed"); }
  *out = w;
  return CAI_OK;
}

extern "C" int cai_qw_destroy(cai_qw_t w)
{
  CAI_ENTER();
  if (!w) return CAI_OK;
  if (ctx().ready) (void)hipStreamSynchronize(ctx().stream);
  qw_free(w);
  return CAI_OK;
}

extern "C" int cai_qw_info(cai_qw_t w, int* qtype, int64_t* rows, int64_t* cols, int64_t* device_bytes)
{
  CAI_ENTER();
  CAI_REQUIRE(w, "cai_qw_info: null weight");
  if (qtype) *qtype = w->qtype;
  if (rows) *rows = w->rows;
  if (cols) *cols = w->cols;
  if (device_bytes) *device_bytes = w->data_bytes + w->aux_bytes + (w->bias ? w->rows * 4 : 0);
  return CAI_OK;
}

extern "C" int cai_qw_dequant_rows(cai_qw_t w, int64_t row0, int64_t n_rows, float* out, int flags)
{
  CAI_ENTER();
  CAI_READY();
  CAI_REQUIRE(w && out, "cai_qw_dequant_rows: null argument");
  CAI_REQUIRE(row0 >= 0 && n_rows > 0 && row0 + n_rows <= w->rows, "cai_qw_dequant_rows: rows [%lld,+%lld) outside %lld", (long long)row0, (long long)n_rows, (long long)w->rows);
  Context& c = ctx();
  const size_t bytes = (size_t)n_rows * w->cols * 4;
  float* d = out;
  if (!(flags & CAI_Y_DEVICE)) { const int rc = ensure_stage(&c.stage_out, &c.stage_out_cap, bytes); if (rc) return rc; d = (float*)c.stage_out; }
  launch_dequant_rows(w, row0, n_rows, d);
  if (!(flags & CAI_Y_DEVICE)) CAI_HIP(hipMemcpyAsync(out, d, bytes, hipMemcpyDeviceToHost, c.stream));
  CAI_HIP(hipStreamSynchronize(c.stream));
  return CAI_OK;
}

extern "C" int cai_qgemv(cai_qw_t w, const float* x, int n_b, float* y, int act, int flags)
{
  CAI_ENTER();
  CAI_READY();
  CAI_REQUIRE(w && x && y, "cai_qgemv: null argument");
  CAI_REQUIRE(n_b >= 1 && n_b <= 8, "cai_qgemv: n_b %d outside 1..8", n_b);
  CAI_REQUIRE(act >= 0 && act <= 3, "cai_qgemv: activation opcode %d", act);
  Context& c = ctx();
  const size_t xb = (size_t)n_b * w->cols * 4, yb = (size_t)n_b * w->rows * 4;
  const float* dx = x; float* dy = y; int rc;
  if (!(flags & CAI_X_DEVICE)) {
    if ((rc = ensure_stage(&c.stage_in, &c.stage_in_cap, xb))) return rc;
    CAI_HIP(hipMemcpyAsync(c.stage_in, x, xb, hipMemcpyHostToDevice, c.stream));
    dx = (const float*)c.stage_in;
  }
  if (!(flags & CAI_Y_DEVICE)) { if ((rc = ensure_stage(&c.stage_out, &c.stage_out_cap, yb))) return rc; dy = (float*)c.stage_out; }
  // A batch on a matrix too large for the cache: the VALU kernel would be compute-bound, the matrix-core kernel streams
  // the weights once for the batch.  Small matrices stay on the single-launch kernel (three launches cost more there).
  if (n_b >= 2 && act == CAI_ACT_NONE && nb_supported(w) && w->data_bytes >= ((int64_t)16 << 20)) {
    if ((rc = nb_linear(w, dx, w->cols, nullptr, 0.0f, n_b, dy, w->rows, nullptr))) return rc;
  } else if ((rc = launch_gemv(w, 0, w->rows, dx, n_b, dy, w->rows, act, nullptr))) return rc;
  CAI_HIP(hipGetLastError());
  if (!(flags & CAI_Y_DEVICE)) {
    CAI_HIP(hipMemcpyAsync(y, dy, yb, hipMemcpyDeviceToHost, c.stream));
    CAI_HIP(hipStreamSynchronize(c.stream));
  }
  return CAI_OK;
}

extern "C" int cai_ffn_gateup(cai_qw_t w, const float* x, const float* gain, float eps, int n_b, float* y, int flags)
{
  CAI_ENTER();
  CAI_READY();
  CAI_REQUIRE(w && x && y, "cai_ffn_gateup: null argument");
  CAI_REQUIRE(n_b >= 1 && n_b <= 8, "cai_ffn_gateup: n_b %d outside 1..8", n_b);
  CAI_REQUIRE(w->rows % 2 == 0, "cai_ffn_gateup: %lld rows is not an up|gate pair", (long long)w->rows);
  Context& c = ctx();
  const int64_t I = w->rows / 2;
  const size_t xb = (size_t)n_b * w->cols * 4, gb = gain ? (size_t)w->cols * 4 : 0, yb = (size_t)n_b * I * 4;
  const float* dx = x; const float* dg = gain; float* dy = y; int rc;
  if (!(flags & CAI_X_DEVICE)) {
    if ((rc = ensure_stage(&c.stage_in, &c.stage_in_cap, xb + gb))) return rc;
    CAI_HIP(hipMemcpyAsync(c.stage_in, x, xb, hipMemcpyHostToDevice, c.stream));
    dx = (const float*)c.stage_in;
    if (gain) {
      CAI_HIP(hipMemcpyAsync((char*)c.stage_in + xb, gain, gb, hipMemcpyHostToDevice, c.stream));
      dg = (const float*)((char*)c.stage_in + xb);
    }
  }
  if (!(flags & CAI_Y_DEVICE)) { if ((rc = ensure_stage(&c.stage_out, &c.stage_out_cap, yb))) return rc; dy = (float*)c.stage_out; }
  MultiGemv m{}; m.n = 1; m.w[0] = w; m.rows[0] = w->rows;
  if ((rc = launch_gemv_multi(m, dx, n_b, dy, I, CAI_ACT_NONE, nullptr, dg, eps, (int)I))) return rc;
  if (!(flags & CAI_Y_DEVICE)) {
    CAI_HIP(hipMemcpyAsync(y, dy, yb, hipMemcpyDeviceToHost, c.stream));
    CAI_HIP(hipStreamSynchronize(c.stream));
  }
  return CAI_OK;
}
