// C entry points of the attention core: validate and route to the MFMA flash
// kernels (bf16 at head size 64; bf16 / fp16 at head sizes 96 and 128) when they cover
// the problem, to the window or generic kernels otherwise.
#include <initializer_list>

#include "jg_common.h"

namespace jg {
bool attn_generic_supported(int d);
int attn_generic_fwd(void* out, float* lse, const void* q, const void* k, const void* v,
                     long long batch, int sq, int sk, int d, float scale, const float* bias,
                     long long bias_period, int dtype, hipStream_t s);
int attn_generic_bwd(void* dq, void* dk, void* dv, float* delta, float* dbias, const void* dout,
                     const void* q, const void* k, const void* v, const void* out,
                     const float* lse, long long batch, int sq, int sk, int d, float scale,
                     const float* bias, long long bias_period, int dtype, hipStream_t s);
bool attn_mfma_fwd_supported(long long batch, int sq, int sk, int d, int dtype, bool has_bias);
int attn_mfma_fwd(void* out, float* lse, const void* q, const void* k, const void* v,
                  long long batch, int sq, int sk, float scale, float* out_acc, float* lse_acc,
                  hipStream_t s);
bool attn_mfma_bwd_supported(long long batch, int sq, int sk, int d, int dtype, bool has_bias);
size_t attn_mfma_bwd_workspace(long long batch, int sq, int sk);
int attn_mfma_bwd(void* dq, void* dk, void* dv, const void* dout, const void* q, const void* k,
                  const void* v, const void* out, const float* lse, long long batch, int sq,
                  int sk, float scale, void* ws, hipStream_t s);
int attn_mfma_bwd_chunks(void* dq, void* const* dk, void* const* dv, const void* dout, const void* q,
                         const void* const* k, const void* const* v, int nchunks, const void* out, const float* lse,
                         long long batch, int sq, int sk, float scale, void* ws, hipStream_t s);
bool attn_wide_supported(long long batch, int sq, int sk, int d, int dtype, bool has_bias);
int attn_wide_fwd(void* out, float* lse, const void* q, const void* k, const void* v, long long batch,
                  int sq, int sk, int d, int dtype, float scale, float* out_acc, float* lse_acc,
                  hipStream_t s);
int attn_wide_bwd(void* dq, void* dk, void* dv, const void* dout, const void* q, const void* k,
                  const void* v, const void* out, const float* lse, long long batch, int sq, int sk,
                  int d, int dtype, float scale, void* ws, hipStream_t s);
bool attn_f32_mfma_fwd_supported(long long batch, int sq, int sk, int d, int dtype, bool has_bias);
int attn_f32_mfma_fwd(void* out, float* lse, const void* q, const void* k, const void* v, long long batch, int sq,
                      int sk, int d, float scale, float* out_acc, float* lse_acc, hipStream_t s);
bool attn_f32_mfma_bwd_supported(long long batch, int sq, int sk, int d, int dtype, bool has_bias);
int attn_f32_mfma_bwd(void* dq, void* dk, void* dv, const void* dout, const void* q, const void* k, const void* v,
                      const void* out, const float* lse, long long batch, int sq, int sk, int d, float scale,
                      void* workspace, hipStream_t s);
bool attn_window_supported(long long batch, int sq, int sk, int d, int dtype);
int attn_window_fwd(void* out, float* lse, const void* q, const void* k, const void* v,
                    long long batch, float scale, const float* bias, long long bias_period,
                    hipStream_t s);
int attn_window_bwd(void* dq, void* dk, void* dv, float* dbias, const void* dout, const void* q,
                    const void* k, const void* v, const void* out, const float* lse,
                    long long batch, float scale, const float* bias, long long bias_period,
                    hipStream_t s);
}  // namespace jg

namespace {
bool known(int dt) { return dt == JG_F32 || dt == JG_BF16 || dt == JG_F16; }

int check_shape(const char* who, int64_t batch, int64_t sq, int64_t sk, int64_t d, float scale,
                int dtype) {
  JG_REQUIRE(known(dtype), "%s: unknown dtype %d", who, dtype);
  JG_REQUIRE(batch >= 0 && sq >= 0 && sk >= 1 && d >= 1, "%s: bad shape", who);
  JG_REQUIRE(sq < (1ll << 30) && sk < (1ll << 30), "%s: sequence too long", who);
  JG_REQUIRE(scale > 0.0f, "%s: scale must be positive", who);
  return JG_OK;
}

// The window kernels move 16 bytes per lane.
bool aligned16(std::initializer_list<const void*> ptrs) {
  for (const void* q : ptrs)
    if ((reinterpret_cast<uintptr_t>(q) & 15) != 0) return false;
  return true;
}
}  // namespace

extern "C" int jg_attn_fwd(void* out, float* lse, const void* q, const void* k, const void* v,
                           int64_t batch, int64_t sq, int64_t sk, int64_t d, float scale,
                           const float* bias, int64_t bias_period, float* out_acc,
                           float* lse_acc, int dtype, void* stream) {
  const char* who = "jg_attn_fwd";
  int rc = check_shape(who, batch, sq, sk, d, scale, dtype);
  if (rc) return rc;
  JG_REQUIRE(q && k && v, "%s: NULL input", who);
  JG_REQUIRE((out_acc == nullptr) == (lse_acc == nullptr),
             "%s: out_acc and lse_acc go together", who);
  JG_REQUIRE(out_acc != nullptr || (out != nullptr && lse != nullptr),
             "%s: nowhere to write the result", who);
  JG_REQUIRE(bias == nullptr || bias_period >= 1, "%s: bias_period must be >= 1", who);
  if (batch == 0 || sq == 0) return JG_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (jg::attn_mfma_fwd_supported(batch, (int)sq, (int)sk, (int)d, dtype, bias != nullptr))
    return jg::attn_mfma_fwd(out, lse, q, k, v, batch, (int)sq, (int)sk, scale, out_acc, lse_acc, s);
  if (jg::attn_wide_supported(batch, (int)sq, (int)sk, (int)d, dtype, bias != nullptr) &&
      aligned16({out, q, k, v, out_acc}))
    return jg::attn_wide_fwd(out, lse, q, k, v, batch, (int)sq, (int)sk, (int)d, dtype, scale, out_acc,
                             lse_acc, s);
  if (out_acc == nullptr && jg::attn_window_supported(batch, (int)sq, (int)sk, (int)d, dtype) &&
      aligned16({out, q, k, v, bias}))
    return jg::attn_window_fwd(out, lse, q, k, v, batch, scale, bias, bias_period, s);
  if (jg::attn_f32_mfma_fwd_supported(batch, (int)sq, (int)sk, (int)d, dtype, bias != nullptr) &&
      aligned16({out, q, k, v, out_acc}))
    return jg::attn_f32_mfma_fwd(out, lse, q, k, v, batch, (int)sq, (int)sk, (int)d, scale, out_acc, lse_acc, s);
  if (!jg::attn_generic_supported((int)d))
    JG_FAIL(JG_ERR_UNSUPPORTED, "%s: head size %lld not in {8, 16, 32, 64, 96, 128}", who, (long long)d);
  if (out_acc != nullptr)
    JG_FAIL(JG_ERR_UNSUPPORTED,
            "%s: the fused merge needs an MFMA path (bf16 with d in {64, 96, 128} or fp16 with d in {96, 128},"
            " sq %% 128 == 0, sk %% 128 == 0; fp32 with d in {32, 64, 128}, no bias);"
            " call jg_lse_merge after the core instead", who);
  rc = jg::attn_generic_fwd(out, lse, q, k, v, batch, (int)sq, (int)sk, (int)d, scale, bias,
                            bias_period, dtype, s);
  if (rc) return rc;
  return JG_OK;
}

extern "C" size_t jg_attn_bwd_workspace_bytes(int64_t batch, int64_t sq, int64_t sk, int64_t d) {
  if (batch <= 0 || sq <= 0) return 0;
  (void)sk;
  (void)d;
  // delta (batch, sq) fp32; the MFMA path needs nothing beyond it
  return (size_t)batch * (size_t)sq * sizeof(float);
}

extern "C" int jg_attn_bwd(void* dq, void* dk, void* dv, const void* dout, const void* q,
                           const void* k, const void* v, const void* out, const float* lse,
                           int64_t batch, int64_t sq, int64_t sk, int64_t d, float scale,
                           const float* bias, int64_t bias_period, float* dbias, int dtype,
                           void* workspace, size_t workspace_bytes, void* stream) {
  const char* who = "jg_attn_bwd";
  int rc = check_shape(who, batch, sq, sk, d, scale, dtype);
  if (rc) return rc;
  JG_REQUIRE(dq && dk && dv && dout && q && k && v && out && lse, "%s: NULL pointer", who);
  JG_REQUIRE(bias == nullptr || bias_period >= 1, "%s: bias_period must be >= 1", who);
  if (batch == 0 || sq == 0) return JG_OK;
  if (workspace == nullptr || workspace_bytes < jg_attn_bwd_workspace_bytes(batch, sq, sk, d))
    JG_FAIL(JG_ERR_WORKSPACE, "%s: workspace %zu < %zu bytes", who, workspace_bytes,
            jg_attn_bwd_workspace_bytes(batch, sq, sk, d));
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dbias == nullptr &&
      jg::attn_mfma_bwd_supported(batch, (int)sq, (int)sk, (int)d, dtype, bias != nullptr))
    return jg::attn_mfma_bwd(dq, dk, dv, dout, q, k, v, out, lse, batch, (int)sq, (int)sk, scale,
                             workspace, s);
  if (dbias == nullptr &&
      jg::attn_wide_supported(batch, (int)sq, (int)sk, (int)d, dtype, bias != nullptr) &&
      aligned16({dq, dk, dv, dout, q, k, v, out}))
    return jg::attn_wide_bwd(dq, dk, dv, dout, q, k, v, out, lse, batch, (int)sq, (int)sk, (int)d,
                             dtype, scale, workspace, s);
  if (jg::attn_window_supported(batch, (int)sq, (int)sk, (int)d, dtype) &&
      aligned16({dq, dk, dv, dout, q, k, v, out, bias, dbias}))
    return jg::attn_window_bwd(dq, dk, dv, dbias, dout, q, k, v, out, lse, batch, scale, bias,
                               bias_period, s);
  if (dbias == nullptr && jg::attn_f32_mfma_bwd_supported(batch, (int)sq, (int)sk, (int)d, dtype, bias != nullptr) &&
      aligned16({dq, dk, dv, dout, q, k, v, out}))
    return jg::attn_f32_mfma_bwd(dq, dk, dv, dout, q, k, v, out, lse, batch, (int)sq, (int)sk, (int)d, scale,
                                 workspace, s);
  if (!jg::attn_generic_supported((int)d))
    JG_FAIL(JG_ERR_UNSUPPORTED, "%s: head size %lld not in {8, 16, 32, 64, 96, 128}", who, (long long)d);
  return jg::attn_generic_bwd(dq, dk, dv, static_cast<float*>(workspace), dbias, dout, q, k, v, out,
                              lse, batch, (int)sq, (int)sk, (int)d, scale, bias, bias_period, dtype,
                              s);
}

extern "C" int jg_attn_bwd_chunks(void* dq, void* const* dk, void* const* dv, const void* dout, const void* q,
                                  const void* const* k, const void* const* v, int64_t n_chunks, const void* out,
                                  const float* lse, int64_t batch, int64_t sq, int64_t sk, int64_t d, float scale,
                                  int dtype, void* workspace, size_t workspace_bytes, void* stream) {
  const char* who = "jg_attn_bwd_chunks";
  int rc = check_shape(who, batch, sq, sk, d, scale, dtype);
  if (rc) return rc;
  JG_REQUIRE(n_chunks >= 1, "%s: n_chunks must be at least 1", who);
  JG_REQUIRE(dq && dk && dv && dout && q && k && v && out && lse, "%s: NULL pointer", who);
  if (n_chunks > 16 || !jg::attn_mfma_bwd_supported(batch, (int)sq, (int)sk, (int)d, dtype, false))
    JG_FAIL(JG_ERR_UNSUPPORTED, "%s: bf16, d = 64, sq and sk multiples of 128 and at most 16 chunks", who);
  for (int64_t c = 0; c < n_chunks; ++c)
    JG_REQUIRE(k[c] && v[c] && dk[c] && dv[c], "%s: NULL pointer for chunk %lld", who, (long long)c);
  if (batch == 0 || sq == 0) return JG_OK;
  if (workspace == nullptr || workspace_bytes < jg_attn_bwd_workspace_bytes(batch, sq, sk, d))
    JG_FAIL(JG_ERR_WORKSPACE, "%s: workspace %zu < %zu bytes", who, workspace_bytes,
            jg_attn_bwd_workspace_bytes(batch, sq, sk, d));
  return jg::attn_mfma_bwd_chunks(dq, dk, dv, dout, q, k, v, (int)n_chunks, out, lse, batch, (int)sq, (int)sk, scale,
                                  workspace, static_cast<hipStream_t>(stream));
}
