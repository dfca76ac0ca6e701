// Geometry shared by the convolution kernels.
#pragma once
#include "jg_common.h"

namespace jg {

// Resolved geometry; 1-D and 2-D problems carry leading axes of extent 1.
struct ConvGeom {
  long long batch;
  int cin, cout;  // channels of the whole tensors
  int groups;     // cin and cout divide into `groups` independent blocks (F.conv's groups)
  int in[3];   // input spatial extent (the padded tile)
  int out[3];  // output spatial extent
  int k[3], s[3], p[3], d[3];
};

// Validate a jg_conv_desc and resolve it. Returns JG_OK or a negative status.
int resolve_conv(const jg_conv_desc* desc, const char* who, ConvGeom* out);

// Direct kernels (conv_direct.hip).
size_t direct_wgrad_workspace(const ConvGeom& g);
int direct_fwd(void* y, const void* x, const void* w, const void* bias, const ConvGeom& g,
               int dtype, hipStream_t s);
int direct_dgrad(void* gx, const void* w, const void* go, const ConvGeom& g, int dtype,
                 hipStream_t s);
int direct_wgrad(void* gw, const void* x, const void* go, const ConvGeom& g, int dtype, void* ws,
                 size_t ws_bytes, hipStream_t s);

// Implicit-GEMM MFMA kernels (conv_mfma.hip). `*_supported` says whether a
// geometry / dtype is covered; the workspace queries return bytes.
bool mfma_fwd_supported(const ConvGeom& g, int dtype);
bool mfma_dgrad_supported(const ConvGeom& g, int dtype);
bool mfma_wgrad_supported(const ConvGeom& g, int dtype);
size_t mfma_fwd_workspace(const ConvGeom& g, int dtype = JG_BF16);
size_t mfma_dgrad_workspace(const ConvGeom& g, int dtype = JG_BF16);
size_t mfma_wgrad_workspace(const ConvGeom& g, int dtype = JG_BF16);
int mfma_fwd(void* y, const void* x, const void* w, const void* bias, const ConvGeom& g,
             void* ws, size_t ws_bytes, hipStream_t s, int dtype = JG_BF16);
// Framed input: x_frame has the padded geometry g.in but only a frame near its edges holds
// data (mfma_frame_bands); the own tile xt sits at [tlo, tlo + tn) inside it.
int mfma_fwd_framed(void* y, const void* x_frame, const void* xt, const int tlo[3], const int tn[3],
                    const void* w, const void* bias, const ConvGeom& g, void* ws, size_t ws_bytes,
                    hipStream_t s);
bool mfma_wgrad_frame_ok(const ConvGeom& g, const int tlo[3], const int tn[3]);
void mfma_frame_bands(const ConvGeom& g, const int tlo[3], const int tn[3], int band_lo[3], int band_hi[3]);
int mfma_dgrad(void* gx, const void* w, const void* go, const ConvGeom& g, void* ws,
               size_t ws_bytes, hipStream_t s, int dtype = JG_BF16);
// Input gradient split between the unpadded tile and the neighbours' strips: the produced
// (padded) tensor has extent g.in; [lo, lo + n) of it is the tile.
int mfma_dgrad_fold(void* gx, void* const strips[27], const int lo[3], const int n[3], const void* w,
                    const void* go, const ConvGeom& g, void* ws, size_t ws_bytes, hipStream_t s);
// gb (Cout,) or NULL: the bias gradient from the same pass over go
// xt / tlo / tn: framed input as for mfma_fwd_framed, or NULL
int mfma_wgrad(void* gw, void* gb, const void* x, const void* go, const ConvGeom& g, void* ws,
               size_t ws_bytes, hipStream_t s, const void* xt = nullptr, const int* tlo = nullptr,
               const int* tn = nullptr, int dtype = JG_BF16);
// dst (batch, parts, per_batch) bf16 = the bf16 parts of src (batch, per_batch), whose sum is src:
// three for fp32, two for fp16. The operand layout of the split mode of the MFMA kernels.
int split_parts_bf16(uint16_t* dst, const void* src, int src_dtype, size_t batch, size_t per_batch, hipStream_t s);

}  // namespace jg
