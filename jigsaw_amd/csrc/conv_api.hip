// C entry points of the local convolution: validate, resolve the geometry and
// route to the implicit-GEMM MFMA kernels when they cover the problem, to the
// direct kernels otherwise.
#include "conv_common.h"

namespace jg {

int resolve_conv(const jg_conv_desc* d, const char* who, ConvGeom* out) {
  JG_REQUIRE(d != nullptr, "%s: desc is NULL", who);
  JG_REQUIRE(d->n_spatial >= 1 && d->n_spatial <= 3, "%s: n_spatial %d not in 1..3", who,
             d->n_spatial);
  JG_REQUIRE(d->batch >= 0 && d->c_in >= 1 && d->c_out >= 1, "%s: bad batch / channels", who);
  JG_REQUIRE(d->groups >= 1 && d->c_in % d->groups == 0 && d->c_out % d->groups == 0,
             "%s: groups = %d must divide the channels (%d in, %d out)", who, d->groups, d->c_in, d->c_out);
  ConvGeom g;
  g.groups = d->groups;
  g.batch = d->batch;
  g.cin = d->c_in;
  g.cout = d->c_out;
  const int lead = 3 - d->n_spatial;
  for (int a = 0; a < 3; ++a) {
    if (a < lead) {
      g.in[a] = 1; g.k[a] = 1; g.s[a] = 1; g.p[a] = 0; g.d[a] = 1;
    } else {
      g.in[a] = d->in_size[a]; g.k[a] = d->kernel[a]; g.s[a] = d->stride[a];
      g.p[a] = d->padding[a]; g.d[a] = d->dilation[a];
    }
    JG_REQUIRE(g.in[a] >= 1 && g.k[a] >= 1 && g.s[a] >= 1 && g.p[a] >= 0 && g.d[a] >= 1,
               "%s: bad geometry on axis %d (in %d, k %d, s %d, p %d, d %d)", who, a, g.in[a],
               g.k[a], g.s[a], g.p[a], g.d[a]);
    const int span = g.in[a] + 2 * g.p[a] - g.d[a] * (g.k[a] - 1) - 1;
    JG_REQUIRE(span >= 0, "%s: kernel extent exceeds the padded input on axis %d", who, a);
    g.out[a] = span / g.s[a] + 1;
  }
  *out = g;
  return JG_OK;
}

}  // namespace jg

namespace {
bool known(int dt) { return dt == JG_F32 || dt == JG_BF16 || dt == JG_F16; }
}  // namespace

extern "C" size_t jg_conv_workspace_bytes(const jg_conv_desc* desc, int op, int dtype) {
  jg::ConvGeom g;
  if (jg::resolve_conv(desc, "jg_conv_workspace_bytes", &g) != JG_OK) return 0;
  switch (op) {
    case JG_CONV_FWD:
      return jg::mfma_fwd_supported(g, dtype) ? jg::mfma_fwd_workspace(g, dtype) : 0;
    case JG_CONV_DGRAD:
      return jg::mfma_dgrad_supported(g, dtype) ? jg::mfma_dgrad_workspace(g, dtype) : 0;
    case JG_CONV_WGRAD:
      return jg::mfma_wgrad_supported(g, dtype) ? jg::mfma_wgrad_workspace(g, dtype)
                                                : jg::direct_wgrad_workspace(g);
    default:
      return 0;
  }
}

extern "C" int jg_conv_fwd(void* y, const void* x, const void* w, const void* bias,
                           const jg_conv_desc* desc, int dtype, void* workspace,
                           size_t workspace_bytes, void* stream) {
  jg::ConvGeom g;
  int rc = jg::resolve_conv(desc, "jg_conv_fwd", &g);
  if (rc) return rc;
  JG_REQUIRE(y && x && w, "jg_conv_fwd: NULL pointer");
  JG_REQUIRE(known(dtype), "jg_conv_fwd: unknown dtype %d", dtype);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (jg::mfma_fwd_supported(g, dtype)) return jg::mfma_fwd(y, x, w, bias, g, workspace, workspace_bytes, s, dtype);
  return jg::direct_fwd(y, x, w, bias, g, dtype, s);
}

extern "C" int jg_conv_dgrad(void* gx, const void* w, const void* go, const jg_conv_desc* desc,
                             int dtype, void* workspace, size_t workspace_bytes, void* stream) {
  jg::ConvGeom g;
  int rc = jg::resolve_conv(desc, "jg_conv_dgrad", &g);
  if (rc) return rc;
  JG_REQUIRE(gx && w && go, "jg_conv_dgrad: NULL pointer");
  JG_REQUIRE(known(dtype), "jg_conv_dgrad: unknown dtype %d", dtype);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (jg::mfma_dgrad_supported(g, dtype)) return jg::mfma_dgrad(gx, w, go, g, workspace, workspace_bytes, s, dtype);
  return jg::direct_dgrad(gx, w, go, g, dtype, s);
}

extern "C" int jg_conv_dgrad_fold(void* gx, void* const send[27], const void* w, const void* go,
                                  const jg_conv_desc* desc, const jg_halo_geom* geom, int dtype,
                                  void* workspace, size_t workspace_bytes, void* stream) {
  jg::ConvGeom g;
  int rc = jg::resolve_conv(desc, "jg_conv_dgrad_fold", &g);
  if (rc) return rc;
  JG_REQUIRE(gx && send && w && go && geom, "jg_conv_dgrad_fold: NULL pointer");
  JG_REQUIRE(known(dtype), "jg_conv_dgrad_fold: unknown dtype %d", dtype);
  JG_REQUIRE(geom->planes == g.batch * g.cin, "jg_conv_dgrad_fold: geom->planes %lld != batch * c_in %lld",
             (long long)geom->planes, (long long)(g.batch * g.cin));
  int lo[3], n[3];
  for (int a = 0; a < 3; ++a) {
    lo[a] = geom->lo[a];
    n[a] = geom->size[a];
    JG_REQUIRE(lo[a] >= 0 && geom->hi[a] >= 0 && n[a] >= 1 && lo[a] + n[a] + geom->hi[a] == g.in[a],
               "jg_conv_dgrad_fold: axis %d: lo %d + size %d + hi %d != padded extent %d", a, lo[a], n[a],
               geom->hi[a], g.in[a]);
  }
  if (dtype != JG_BF16 || !jg::mfma_dgrad_supported(g, dtype))
    JG_FAIL(JG_ERR_UNSUPPORTED, "jg_conv_dgrad_fold: geometry / dtype only has the unfused path");
  return jg::mfma_dgrad_fold(gx, send, lo, n, w, go, g, workspace, workspace_bytes,
                             static_cast<hipStream_t>(stream));
}

extern "C" int jg_conv_wgrad(void* gw, const void* x, const void* go, const jg_conv_desc* desc,
                             int dtype, void* workspace, size_t workspace_bytes, void* stream) {
  jg::ConvGeom g;
  int rc = jg::resolve_conv(desc, "jg_conv_wgrad", &g);
  if (rc) return rc;
  JG_REQUIRE(gw && x && go, "jg_conv_wgrad: NULL pointer");
  JG_REQUIRE(known(dtype), "jg_conv_wgrad: unknown dtype %d", dtype);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (jg::mfma_wgrad_supported(g, dtype))
    return jg::mfma_wgrad(gw, nullptr, x, go, g, workspace, workspace_bytes, s, nullptr, nullptr, nullptr, dtype);
  return jg::direct_wgrad(gw, x, go, g, dtype, workspace, workspace_bytes, s);
}

namespace {
// Own extent of a framed input inside the padded tensor of `g`; checks the pairing.
int framed_extent(const jg::ConvGeom& g, const jg_halo_geom* geom, const char* who, int tlo[3], int tn[3]) {
  JG_REQUIRE(geom != nullptr, "%s: geom is NULL", who);
  JG_REQUIRE(geom->planes == g.batch * g.cin, "%s: geom->planes %lld != batch * c_in %lld", who,
             (long long)geom->planes, (long long)(g.batch * g.cin));
  for (int a = 0; a < 3; ++a) {
    tlo[a] = geom->lo[a];
    tn[a] = geom->size[a];
    JG_REQUIRE(tlo[a] >= 0 && geom->hi[a] >= 0 && tn[a] >= 1 && tlo[a] + tn[a] + geom->hi[a] == g.in[a],
               "%s: axis %d: lo %d + size %d + hi %d != padded extent %d", who, a, tlo[a], tn[a], geom->hi[a],
               g.in[a]);
  }
  return JG_OK;
}
}  // namespace

extern "C" int jg_conv_frame_bands(const jg_conv_desc* desc, const jg_halo_geom* geom, int dtype,
                                   int32_t band_lo[3], int32_t band_hi[3]) {
  jg::ConvGeom g;
  int rc = jg::resolve_conv(desc, "jg_conv_frame_bands", &g);
  if (rc) return rc;
  JG_REQUIRE(band_lo && band_hi, "jg_conv_frame_bands: NULL pointer");
  int tlo[3], tn[3];
  rc = framed_extent(g, geom, "jg_conv_frame_bands", tlo, tn);
  if (rc) return rc;
  if (dtype != JG_BF16 || !jg::mfma_fwd_supported(g, dtype) || !jg::mfma_wgrad_supported(g, dtype) ||
      !jg::mfma_wgrad_frame_ok(g, tlo, tn))
    JG_FAIL(JG_ERR_UNSUPPORTED, "jg_conv_frame_bands: geometry / dtype has no framed kernels");
  int blo[3], bhi[3];
  jg::mfma_frame_bands(g, tlo, tn, blo, bhi);
  for (int a = 0; a < 3; ++a) {
    band_lo[a] = blo[a];
    band_hi[a] = bhi[a];
  }
  return JG_OK;
}

extern "C" int jg_conv_fwd_framed(void* y, const void* x_frame, const void* x_tile, const void* w,
                                  const void* bias, const jg_conv_desc* desc, const jg_halo_geom* geom,
                                  int dtype, void* workspace, size_t workspace_bytes, void* stream) {
  jg::ConvGeom g;
  int rc = jg::resolve_conv(desc, "jg_conv_fwd_framed", &g);
  if (rc) return rc;
  JG_REQUIRE(y && x_frame && x_tile && w, "jg_conv_fwd_framed: NULL pointer");
  JG_REQUIRE((reinterpret_cast<uintptr_t>(x_tile) & 3) == 0, "jg_conv_fwd_framed: x_tile must be 4-byte aligned");
  JG_REQUIRE(known(dtype), "jg_conv_fwd_framed: unknown dtype %d", dtype);
  int tlo[3], tn[3];
  rc = framed_extent(g, geom, "jg_conv_fwd_framed", tlo, tn);
  if (rc) return rc;
  if (dtype != JG_BF16 || !jg::mfma_fwd_supported(g, dtype) || tn[2] % 2 != 0)
    JG_FAIL(JG_ERR_UNSUPPORTED, "jg_conv_fwd_framed: geometry / dtype has no framed kernel");
  return jg::mfma_fwd_framed(y, x_frame, x_tile, tlo, tn, w, bias, g, workspace, workspace_bytes,
                             static_cast<hipStream_t>(stream));
}

extern "C" int jg_conv_wgrad_framed(void* gw, void* gb, const void* x_frame, const void* x_tile,
                                    const void* go, const jg_conv_desc* desc, const jg_halo_geom* geom,
                                    int dtype, void* workspace, size_t workspace_bytes, void* stream) {
  jg::ConvGeom g;
  int rc = jg::resolve_conv(desc, "jg_conv_wgrad_framed", &g);
  if (rc) return rc;
  JG_REQUIRE(gw && x_frame && x_tile && go, "jg_conv_wgrad_framed: NULL pointer");
  JG_REQUIRE((reinterpret_cast<uintptr_t>(x_tile) & 3) == 0, "jg_conv_wgrad_framed: x_tile must be 4-byte aligned");
  JG_REQUIRE(known(dtype), "jg_conv_wgrad_framed: unknown dtype %d", dtype);
  int tlo[3], tn[3];
  rc = framed_extent(g, geom, "jg_conv_wgrad_framed", tlo, tn);
  if (rc) return rc;
  if (dtype != JG_BF16 || !jg::mfma_wgrad_supported(g, dtype))
    JG_FAIL(JG_ERR_UNSUPPORTED, "jg_conv_wgrad_framed: geometry / dtype has no framed kernel");
  return jg::mfma_wgrad(gw, gb, x_frame, go, g, workspace, workspace_bytes, static_cast<hipStream_t>(stream),
                        x_tile, tlo, tn);
}

extern "C" int jg_conv_wgrad_bias(void* gw, void* gb, const void* x, const void* go,
                                  const jg_conv_desc* desc, int dtype, void* workspace,
                                  size_t workspace_bytes, void* stream) {
  jg::ConvGeom g;
  int rc = jg::resolve_conv(desc, "jg_conv_wgrad_bias", &g);
  if (rc) return rc;
  JG_REQUIRE(gw && gb && x && go, "jg_conv_wgrad_bias: NULL pointer");
  JG_REQUIRE(known(dtype), "jg_conv_wgrad_bias: unknown dtype %d", dtype);
  if (dtype != JG_BF16 || !jg::mfma_wgrad_supported(g, dtype))
    JG_FAIL(JG_ERR_UNSUPPORTED, "jg_conv_wgrad_bias: geometry / dtype only has the separate kernels");
  return jg::mfma_wgrad(gw, gb, x, go, g, workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}
