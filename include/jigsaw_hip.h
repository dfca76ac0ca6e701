/*
 * libjigsaw_hip — C ABI of the MI355X (gfx950) kernels that sit underneath the
 * per-rank hot path of RAI-SCC/jigsaw's domain- and sequence-parallel layers.
 *
 * Conventions
 *   - Every pointer is a device pointer owned by the caller unless it is
 *     documented as a host pointer. The library never allocates, frees or keeps
 *     a pointer past the call.
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream). Calls
 *     only enqueue work; they never synchronise the device.
 *   - Return value: JG_OK (0) or a negative jg_status. jg_last_error() returns
 *     the message of the last failure on the calling host thread.
 *   - Tensors are dense and row-major ("contiguous" in torch terms) in the
 *     layout named per function.
 *   - All functions are re-entrant and may be called from any host thread.
 *
 * The reference has no FFI: its boundary is Python callables held on per-layer
 * config objects. Each entry point cites the reference code it stands in for
 * (paths relative to the reference checkout).
 */
#ifndef JIGSAW_HIP_H
#define JIGSAW_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum { JG_F32 = 0, JG_BF16 = 1, JG_F16 = 2 } jg_dtype;

typedef enum {
  JG_OK = 0,
  JG_ERR_BAD_ARG = -1,     /* a shape / pointer / size argument is invalid        */
  JG_ERR_UNSUPPORTED = -2, /* valid request the kernels do not cover              */
  JG_ERR_LAUNCH = -3,      /* the HIP runtime refused the launch                  */
  JG_ERR_WORKSPACE = -4    /* workspace too small (see the *_workspace query)     */
} jg_status;

/* Message of the most recent failure on this host thread ("" if none). */
const char* jg_last_error(void);
/* ABI version, bumped on any signature change. */
int jg_abi_version(void);

/* ------------------------------------------------------------------------- *
 * Halo movement (bit-exact copies / fixed-order adds; HBM-bound)
 *
 * Geometry of one rank's tile. Spatial axes are (D, H, W); a 2-D tile has
 * size[0] = 1 and lo[0] = hi[0] = 0. `planes` = batch * channels (the tensors
 * are channels-first, so each plane is one contiguous (D, H, W) block).
 * lo / hi are the halo widths in front of / behind the interior on each axis:
 * for jigsaw's span [lo_g, lo_g + need) of needed_input_span
 * (jigsaw/modules/convolution/_conv/halo.py:9-63) they are
 * lo = r*n - lo_g and hi = lo_g + need - (r+1)*n.
 *
 * Neighbour tables have 27 slots indexed (dd+1)*9 + (dh+1)*3 + (dw+1) for the
 * neighbour at offset (dd, dh, dw) in {-1,0,1}^3; slot 13 is this rank. A NULL
 * slot is a neighbour outside the global domain (its halo is zero on assemble,
 * contributes nothing on fold, is skipped on pack). The 2-D entry points take
 * 9 slots indexed (dh+1)*3 + (dw+1), slot 4 = this rank.
 *
 * Strip shapes: the strip of neighbour (dd, dh, dw) is dense
 * (planes, ed, eh, ew) where, per axis and for the three verbs:
 *                      offset -1      offset 0     offset +1
 *   assemble (recv)      lo           size          hi     <- fills my halo
 *   pack_fwd (send)      hi           size          lo     <- their halo of me
 *   pack_bwd (send)      lo           size          hi     <- my halo's grads
 *   fold     (recv)      hi           size          lo     <- their halo of me
 *
 * Where the need spans drift against the tiles (out_local * stride != n,
 * halo.py:49-63) the widths differ from rank to rank. The two verbs marked
 * "their halo of me" then take a geometry with hi = the hi width of the lower
 * neighbour and lo = the lo width of the upper neighbour: jg_halo_pack_3d with
 * from_padded = 0 and jg_halo_fold_border_3d, which read no padded tensor.
 * jg_halo_fold_3d indexes the padded gradient and the strips with one set of
 * widths; for a drifting span call it with an empty strip table (gx = 0 + own)
 * and finish with jg_halo_fold_border_3d.
 * ------------------------------------------------------------------------- */
typedef struct {
  int64_t planes;
  int32_t size[3];
  int32_t lo[3];
  int32_t hi[3];
} jg_halo_geom;

/* x_aug (planes, D+lo+hi, H+lo+hi, W+lo+hi) <- own tile src[13] + 26 strips.
 * One pass over the destination: every element is written exactly once (copied
 * or zero), which replaces new_zeros + narrow().copy_() per split axis in
 * halo_gather (jigsaw/modules/convolution/_conv/halo.py:66-156) and the
 * all_to_all staging of exchange_along_axis (_common/halo.py:7-63).
 * elem_size is 2 or 4 bytes; bytes are moved untouched (-0.0 and NaN payloads
 * survive). */
int jg_halo_assemble_3d(void* x_aug, const void* const src[27],
                        const jg_halo_geom* geom, int elem_size, void* stream);
int jg_halo_assemble_2d(void* x_aug, const void* const src[9], int64_t planes,
                        int H, int W, int lo_h, int hi_h, int lo_w, int hi_w,
                        int elem_size, void* stream);

/* jg_halo_assemble_3d restricted to a frame: only the cells whose padded
 * coordinate on some axis lies in the first band_lo[axis] or the last
 * band_hi[axis] positions are written, the rest of x_aug is left untouched. For
 * the framed convolution entry points, which read the tile itself wherever their
 * window stays inside it and x_aug only near the edges (bands from
 * jg_conv_frame_bands). */
int jg_halo_assemble_frame_3d(void* x_aug, const void* const src[27],
                              const jg_halo_geom* geom, const int32_t band_lo[3],
                              const int32_t band_hi[3], int elem_size, void* stream);

/* Cut the strips this rank sends. from_padded = 0: `src` is the own tile
 * (planes, D, H, W) and strip (dd,dh,dw) is the edge block that neighbour needs
 * for its halo (forward; the x.narrow(axis, col, sn) sends of halo.py:134-147).
 * from_padded = 1: `src` is a padded tensor (planes, D+.., H+.., W+..) and strip
 * (dd,dh,dw) is the halo block that neighbour owns (backward; the
 * g_x_need.narrow sends of halo.py:222-226). NULL slots are skipped. */
int jg_halo_pack_3d(void* const strips[27], const void* src,
                    const jg_halo_geom* geom, int from_padded, int elem_size,
                    void* stream);
int jg_halo_pack_2d(void* const strips[9], const void* src, int64_t planes,
                    int H, int W, int lo_h, int hi_h, int lo_w, int hi_w,
                    int from_padded, int elem_size, void* stream);

/* gx (planes, D, H, W) <- fold of the padded gradient gx_aug and the strips the
 * neighbours sent back. Restates halo_scatter_add (halo.py:159-251) applied in
 * reverse axis order W, H, D (distributed.py:378-389) with its exact
 * association: per axis acc = 0; acc += lower neighbour; acc += own;
 * acc += upper neighbour, each add rounded to `dtype`; the W fold is innermost.
 * Needs lo <= size and hi <= size on every axis. */
int jg_halo_fold_3d(void* gx, const void* gx_aug, const void* const strips[27],
                    const jg_halo_geom* geom, int dtype, void* stream);
int jg_halo_fold_2d(void* gx, const void* gx_aug, const void* const strips[9],
                    int64_t planes, int H, int W, int lo_h, int hi_h, int lo_w,
                    int hi_w, int dtype, void* stream);

/* Second half of a fold whose own contributions are already in place: gx
 * (planes, D, H, W) holds `0 + own` in every cell (what jg_conv_dgrad_fold
 * writes) and the cells a neighbour reaches get the neighbours' strips added, in
 * place, in the order of jg_halo_fold_3d (halo.py:207-249,
 * distributed.py:378-389). Together with jg_conv_dgrad_fold this gives the same
 * bits as jg_conv_dgrad + jg_halo_pack_3d(from_padded) + jg_halo_fold_3d without
 * the padded gradient ever reaching memory. */
int jg_halo_fold_border_3d(void* gx, const void* const strips[27],
                           const jg_halo_geom* geom, int dtype, void* stream);

/* Halo exchange along ONE split axis for need spans of any shape - spans that leave out rows
 * the rank owns, or that reach ranks which are not adjacent (the fused entry points above cover
 * spans that hold the owned rows and reach one tile to either side at most). A tensor is seen as
 * (outer, rows, inner) around the axis; a segment is `count` rows [src_start, +count) of `src`
 * (outer, src_rows, inner) that belong at rows [dst_start, +count) of the destination.
 * jg_halo_axis_gather: dst (outer, dst_rows, inner) = zero, then every segment copied in (bytes
 * untouched; a later segment overwrites an earlier one): the need span from the own tile and the
 * peers' parts (x_need = zeros; x_need[off : off + cnt] = part, _conv/halo.py:112-114, 134-154),
 * or, with one segment, the contiguous part cut for a peer (:140-147, 222-226).
 * jg_halo_axis_scatter_add: dst = 0, then dst[dst_start : +count] += segment for the segments IN
 * THE ORDER GIVEN, each sum rounded to `dtype` (g_local = zeros; g_local[...] += recv[peer] for
 * peer = 0 .. G-1, _conv/halo.py:207, 247-249): bit-identical to the reference's loop.
 * At most JG_HALO_AXIS_MAX_SEGMENTS segments a call (JG_ERR_BAD_ARG beyond). */
#define JG_HALO_AXIS_MAX_SEGMENTS 16
typedef struct jg_axis_segment {
  const void* src;
  int64_t src_rows;
  int64_t src_start;
  int64_t dst_start;
  int64_t count;
} jg_axis_segment;
int jg_halo_axis_gather(void* dst, int64_t outer, int64_t dst_rows, int64_t inner,
                        const jg_axis_segment* segs, int n_segs, int elem_size, void* stream);
int jg_halo_axis_scatter_add(void* dst, int64_t outer, int64_t dst_rows, int64_t inner,
                             const jg_axis_segment* segs, int n_segs, int dtype, void* stream);

/* ------------------------------------------------------------------------- *
 * DistributedRoll (pure copies; HBM-bound)
 * ------------------------------------------------------------------------- */

/* dst = torch.roll(src, shifts, dims) for a dense tensor of `ndim` <= 6 axes
 * (jigsaw/modules/roll/_distributed_roll.py:99). shifts[i] is the shift of axis
 * i (0 = not rolled), any sign, taken modulo sizes[i]. dst must not alias src. */
int jg_roll(void* dst, const void* src, int ndim, const int64_t* sizes,
            const int64_t* shifts, int elem_size, void* stream);

/* The wrapped slab of exchange_halo_1d (_distributed_roll.py:44-48, 59): with
 * window > 0 the leading `window` entries of `axis`, else the trailing
 * |window|. jg_roll_pack copies that slab of x into the dense `strip`
 * (x[sl].contiguous()); jg_roll_unpack writes a dense strip into that slab of x
 * in place (x[sl] = recv). */
int jg_roll_pack(void* strip, const void* x, int ndim, const int64_t* sizes,
                 int axis, int64_t window, int elem_size, void* stream);
int jg_roll_unpack(void* x, const void* strip, int ndim, const int64_t* sizes,
                   int axis, int64_t window, int elem_size, void* stream);

/* The steps of distributed_roll (_distributed_roll.py:63-113) folded into one pass each.
 * jg_roll_pack_fused: jg_roll, then jg_roll_pack of the rolled tensor along `axis`, then the
 * clearing of `clear` (the buffer the neighbour's slab is received in; may be NULL): lines 99 and
 * 44-49. jg_roll_unpack_pack: jg_roll_unpack of the slab received along axis1, then
 * jg_roll_pack along axis2 of the tensor so updated, then the clearing of clear2: line 59 of one
 * exchange and 44-49 of the next. Both need 16-byte aligned tensors whose trailing axes (behind
 * the slab axes, not rolled) span a multiple of 16 bytes; JG_ERR_UNSUPPORTED otherwise. */
int jg_roll_pack_fused(void* dst, void* strip, void* clear, const void* src, int ndim, const int64_t* sizes,
                       const int64_t* shifts, int axis, int64_t window, int elem_size, void* stream);
int jg_roll_unpack_pack(void* x, const void* recv1, int axis1, int64_t window1, void* strip2, void* clear2,
                        int axis2, int64_t window2, int ndim, const int64_t* sizes, int elem_size, void* stream);

/* ------------------------------------------------------------------------- *
 * Sharded LayerNorm (last axis split over the channel group; HBM-bound)
 *
 * x is (rows, cols) dense with cols = the LOCAL width. Statistics are fp32.
 * The two all-reduces between partial statistics and apply stay with the
 * caller (jigsaw/modules/normalization/_functional.py:49-53, 160-171).
 * ------------------------------------------------------------------------- */

/* Per row: mean[r] = mean(x[r,:]), var[r] = biased variance of x[r,:]
 * (local_mean / local_var of _functional.py:46-47). */
int jg_ln_partial_fwd(float* mean, float* var, const void* x, int64_t rows,
                      int64_t cols, int x_dtype, void* stream);

/* x_hat = (x - mean) / sqrt(var + eps);  y = w * x_hat + b  (_functional.py:55-58)
 * with the COMBINED statistics. Also writes std[r] = sqrt(var[r] + eps), the
 * tensor the backward saves (_functional.py:75). w, b, y, x_hat have dtype
 * out_dtype; b may be NULL; x_hat may be NULL (inference). */
int jg_ln_apply(void* y, void* x_hat, float* std_out, const void* x,
                const float* mean, const float* var, const void* w, const void* b,
                int64_t rows, int64_t cols, float eps, int x_dtype, int out_dtype,
                void* stream);

/* Backward partials (_functional.py:150-168), one pass over g and x_hat:
 *   mean_gxn[r] = mean_c(g*w), dot_gxn_xhat[r] = sum_c(g*w*x_hat)   (per row)
 *   gw[c] = sum_r g*x_hat,      gb[c] = sum_r g                     (per column)
 * gw / gb are fp32 (cols,); either may be NULL. workspace: device scratch of
 * jg_ln_bwd_workspace_bytes(rows, cols) bytes (deterministic two-stage column
 * reduction, no atomics). g, x_hat, w share `dtype`. */
size_t jg_ln_bwd_workspace_bytes(int64_t rows, int64_t cols);
int jg_ln_partial_bwd(float* mean_gxn, float* dot_gxn_xhat, float* gw, float* gb,
                      const void* g, const void* x_hat, const void* w, int64_t rows,
                      int64_t cols, int dtype, void* workspace, size_t workspace_bytes,
                      void* stream);

/* jg_ln_partial_bwd without a workspace argument, for callers that cannot allocate
 * device memory (code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc). No counterpart in the reference. Same kernels, same results, same
 * arguments otherwise; the column partials go to a device array built into the library
 * (JG_LN_BWD_STATIC_SCRATCH_BYTES per GPU, held until the process ends). The call
 * allocates and frees nothing. Limits: jg_ln_bwd_workspace_bytes(rows, cols) must fit
 * that array when gw or gb is asked for (min(ceil(rows / 4), 1024) * 2 * cols * 4 bytes:
 * any row count up to 1024 local columns) - JG_ERR_WORKSPACE otherwise; calls on one GPU
 * share the array, so two calls that overlap in time on one GPU (different streams or
 * host threads) race: serialise them. The first call on a device resolves the array's
 * address and must happen outside a stream capture. */
#define JG_LN_BWD_STATIC_SCRATCH_BYTES (8u << 20)
int jg_ln_partial_bwd_static(float* mean_gxn, float* dot_gxn_xhat, float* gw, float* gb,
                             const void* g, const void* x_hat, const void* w, int64_t rows,
                             int64_t cols, int dtype, void* stream);

/* gx = (1/std) * (g*w - mean_gxn - x_hat * dot_gxn_xhat / n_global) with the
 * COMBINED row terms (_functional.py:173-175). */
int jg_ln_bwd_apply(void* gx, const void* g, const void* x_hat, const void* w,
                    const float* mean_gxn, const float* dot_gxn_xhat,
                    const float* std, int64_t rows, int64_t cols, int64_t n_global,
                    int dtype, void* stream);

/* LayerNorm over rows that are NOT split over a channel group (nn.LayerNorm as the
 * example Swin block applies it, examples/swin.py:186-188, 209-210): statistics and
 * apply in one pass, y = w * (x - mean) * rstd + b with rstd = 1/sqrt(var + eps)
 * (biased variance), fp32 arithmetic. w, b (may be NULL) are fp32; x and y may
 * differ in dtype when one of them is fp32 (autocast: bf16 in, fp32 or bf16 out).
 * mean, rstd (rows) fp32 are what the backward needs besides x. cols must be a
 * multiple of 8 and at most 2048 (jg_ln_plain_supported), x / y 16-byte aligned;
 * JG_ERR_UNSUPPORTED otherwise: use the partial-statistics entry points above. */
int jg_ln_plain_supported(int64_t cols);
int jg_ln_plain_fwd(void* y, float* mean, float* rstd, const void* x, const float* w,
                    const float* b, int64_t rows, int64_t cols, float eps, int x_dtype,
                    int y_dtype, void* stream);

/* Backward of jg_ln_plain_fwd from (x, mean, rstd): x_hat = (x - mean) * rstd,
 * gx = rstd * (g w - mean_c(g w) - x_hat * mean_c(g w x_hat)) in x's dtype (gx may
 * be NULL), gw[c] = sum_r g x_hat, gb[c] = sum_r g (fp32, either may be NULL;
 * two-stage deterministic column sums through the workspace). */
size_t jg_ln_plain_bwd_workspace_bytes(int64_t rows, int64_t cols);
int jg_ln_plain_bwd(void* gx, float* gw, float* gb, const void* g, const void* x,
                    const float* mean, const float* rstd, const float* w, int64_t rows,
                    int64_t cols, int g_dtype, int x_dtype, void* workspace,
                    size_t workspace_bytes, void* stream);
/* jg_ln_plain_bwd with the gradient that reaches x past the normalisation added in:
 * gx = round(gx of jg_ln_plain_bwd) + add, add (rows, cols) in x's dtype. For the pre-norm
 * residual blocks x + f(norm(x)) (examples/swin.py:206-209), where autograd would add the two
 * gradient tensors in a pass of its own. */
int jg_ln_plain_bwd_add(void* gx, float* gw, float* gb, const void* g, const void* x,
                        const float* mean, const float* rstd, const float* w, int64_t rows,
                        int64_t cols, int g_dtype, int x_dtype, void* workspace,
                        size_t workspace_bytes, const void* add, void* stream);

/* ------------------------------------------------------------------------- *
 * GroupNorm over a spatially sharded input (HBM-bound)
 *
 * x (batch, channels, spatial) dense, `spatial` = product of the LOCAL spatial
 * extents; `groups` channel groups of channels / groups consecutive channels,
 * none of which straddles a channel shard. The sums are the rank's partials:
 * the caller adds them up over the spatial process groups (one all-reduce of
 * (count, sum), one of the centred squares; backward one of the two sums),
 * as _GroupNorm does (jigsaw/modules/normalization/_functional.py:317-468).
 * workspace: jg_gn_workspace_bytes(batch, channels, spatial) bytes of device
 * scratch (block partials, added up in a fixed order: deterministic).
 * ------------------------------------------------------------------------- */
size_t jg_gn_workspace_bytes(int64_t batch, int64_t channels, int64_t spatial);

/* sum[n][grp] = sum of x over the group's channels and the local positions
 * (_functional.py:356-359; the count is channels / groups * spatial). */
int jg_gn_partial_sum(float* sum, const void* x, int64_t batch, int64_t channels,
                      int64_t spatial, int64_t groups, int dtype, void* workspace,
                      size_t workspace_bytes, void* stream);

/* sq[n][grp] = sum of (x - mean[n][grp])^2 with the GLOBAL mean: the two-pass
 * variance of _functional.py:364-366. */
int jg_gn_partial_sqdev(float* sq, const void* x, const float* mean, int64_t batch,
                        int64_t channels, int64_t spatial, int64_t groups, int dtype,
                        void* workspace, size_t workspace_bytes, void* stream);

/* x_norm = (x - mean) * rstd, y = x_norm * weight[c] + bias[c]
 * (_functional.py:370-381). weight / bias (channels,) in `dtype`, either may be
 * NULL. mean / rstd fp32 (batch, groups). */
int jg_gn_apply(void* y, void* x_norm, const void* x, const float* mean, const float* rstd,
                const void* weight, const void* bias, int64_t batch, int64_t channels,
                int64_t spatial, int64_t groups, int dtype, void* stream);

/* Backward partials (_functional.py:438-462), one pass over g and x_norm:
 *   gsum[n][grp]  = sum of g * weight[c]            over the group, local positions
 *   gxsum[n][grp] = sum of g * weight[c] * x_norm   "
 *   gw[c] = sum over batch and positions of g * x_norm,  gb[c] = sum of g
 * gw / gb fp32 (channels,), either may be NULL; weight may be NULL (= 1). */
int jg_gn_partial_bwd(float* gsum, float* gxsum, float* gw, float* gb, const void* g,
                      const void* x_norm, const void* weight, int64_t batch,
                      int64_t channels, int64_t spatial, int64_t groups, int dtype,
                      void* workspace, size_t workspace_bytes, void* stream);

/* gx = rstd * (g * weight[c] - gsum / count - x_norm * gxsum / count) with the
 * COMBINED sums and the global element count per (sample, group), fp32
 * (batch, groups) each (_functional.py:465). */
int jg_gn_bwd_apply(void* gx, const void* g, const void* x_norm, const void* weight,
                    const float* rstd, const float* gsum, const float* gxsum,
                    const float* count, int64_t batch, int64_t channels, int64_t spatial,
                    int64_t groups, int dtype, void* stream);

/* ------------------------------------------------------------------------- *
 * Token projections around the attention core, head split / merge fused into
 * the GEMM addressing (MFMA-bound for bf16)
 *
 * Stand in for `self.qkv(x)` + rearrange "... n s (three h d) -> three ... n h s d"
 * and for rearrange "... n h s d -> ... n s (h d)" + `.contiguous()` +
 * `self.head_concat(out)` of DistributedAttention.forward
 * (jigsaw/modules/attention/_attention.py:881-918), and for their backward.
 *
 * A token x feature matrix is either row-major (tokens, features) or, with its
 * *_heads flag set, the dense tensor (t, B, H, S, D): token = b * S + s,
 * feature = (t * H + h) * D + d, B * S = rows, features = t * H * D.
 * fp32 accumulation; all operands share `dtype`.
 * ------------------------------------------------------------------------- */

/* out(r, n) = sum_k a(r, k) * w[n][k] + bias[n];  w (n_out, k_in) row-major,
 * bias (n_out,) or NULL. Forward of both projections; with the transposed
 * weight also the gradient of a projection's input. */
int jg_proj_nt(void* out, const void* a, const void* w, const void* bias, int dtype,
               int64_t rows, int n_out, int k_in, int a_heads, int out_heads,
               int B, int H, int S, int D, void* stream);

/* jg_proj_nt on row-major bf16 operands with an elementwise step of the two-layer MLP of a
 * transformer block folded into the way out (examples/swin.py:190-194: Linear, GELU, Linear and
 * the residual sum around them; the values are the bf16-rounded results a separate pass over
 * the stored tensor would see, arithmetic in fp32). aux has the shape of out.
 *   JG_EPI_GELU  (1): out = y, aux = gelu(y) (erf form); aux is written
 *   JG_EPI_DGELU (2): out = y * gelu'(aux); aux is read (the saved pre-activation)
 *   JG_EPI_ADD   (3): out = y + aux; aux is read (the residual) */
#define JG_EPI_GELU 1
#define JG_EPI_DGELU 2
#define JG_EPI_ADD 3
int jg_proj_nt_fused(void* out, void* aux, int epilogue, const void* a, const void* w, const void* bias, int dtype,
                     int64_t rows, int n_out, int k_in, void* stream);

/* gw[n][c] = sum_r g(r, n) * x(r, c)  (n, c) row-major, and gb[n] = sum_r g(r, n)
 * (gb may be NULL): weight and bias gradient of a projection (torch's
 * Linear backward; g = grad of the projection's output, x = its input).
 * gw and gb have dtype grad_dtype: `dtype`, or JG_F32 (fp32 parameters under
 * autocast: the fp32 sums are stored without a rounding to the operands' dtype).
 * workspace: jg_proj_tn_workspace(rows, n, c) bytes of device scratch (partial
 * sums per token range, added up in a fixed order: deterministic). */
size_t jg_proj_tn_workspace(int64_t rows, int n, int c);
int jg_proj_tn(void* gw, void* gb, const void* g, const void* x, int dtype, int grad_dtype,
               int64_t rows, int n, int c, int g_heads, int x_heads, int B, int H, int S, int D,
               void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------- *
 * Online-softmax / log-sum-exp merge of ring attention (HBM-bound)
 * ------------------------------------------------------------------------- */

/* In place on o1:  w = sigmoid(l2 - l1);  o1 += w * (o2 - o1);
 * l_new = max(l1,l2) + log(1 + exp(-|l1 - l2|)).
 * Stands in for the Triton kernel behind fused_online_softmax_merge_
 * (jigsaw/modules/attention/_functional/_merge_kernel.py:37-82, 88-172).
 * o1 / o2: (b, h, n, d) when bshd == 0, (b, n, h, d) when bshd != 0;
 * l1, l2, l_new: fp32 (b, h, n). l_new must not alias l1 or l2. */
int jg_lse_merge(void* o1, const float* l1, const void* o2, const float* l2,
                 float* l_new, int64_t b, int64_t h, int64_t n, int64_t d, int bshd,
                 int o1_dtype, int o2_dtype, void* stream);

/* ------------------------------------------------------------------------- *
 * Local convolution on the halo-padded tile (MFMA-bound for bf16 / fp16 with
 * wide channels, FMA otherwise)
 *
 * Layouts are torch's: x (N, Cin, *in), w (Cout, Cin, *kernel), y (N, Cout, *out),
 * all dense, one dtype per call; accumulation is fp32. A 1-D / 2-D problem fills
 * the LAST n_spatial entries of the per-axis arrays (leading entries ignored).
 * `padding` is the LOCAL padding of the call: zero on split axes, whose halo is
 * already in x (jigsaw/modules/convolution/_common/spatial_split.py:75-82).
 * out = (in + 2*padding - dilation*(kernel-1) - 1) / stride + 1 per axis.
 * groups >= 1 divides c_in and c_out; w is then (Cout, Cin / groups, *kernel), as
 * torch's. groups > 1 runs the direct kernels (the matrix-core kernels take groups = 1).
 *
 * Workspace: query with jg_conv_workspace_bytes(desc, op, dtype) (op: 0 = fwd,
 * 1 = dgrad, 2 = wgrad); may be 0, then `workspace` may be NULL. Contents are
 * scratch; concurrent calls need distinct workspaces.
 * ------------------------------------------------------------------------- */
typedef struct {
  int32_t n_spatial; /* 1, 2 or 3 */
  int32_t groups;    /* >= 1, divides c_in and c_out */
  int64_t batch;
  int32_t c_in;
  int32_t c_out;
  int32_t in_size[3];
  int32_t kernel[3];
  int32_t stride[3];
  int32_t padding[3];
  int32_t dilation[3];
} jg_conv_desc;

typedef enum { JG_CONV_FWD = 0, JG_CONV_DGRAD = 1, JG_CONV_WGRAD = 2 } jg_conv_op;

size_t jg_conv_workspace_bytes(const jg_conv_desc* desc, int op, int dtype);

/* y = conv(x, w) + bias  — F.conv{1,2,3}d as called at
 * jigsaw/modules/convolution/_conv/channel_comm.py:155-158 (table config.py:27).
 * bias (Cout,) may be NULL. */
int jg_conv_fwd(void* y, const void* x, const void* w, const void* bias,
                const jg_conv_desc* desc, int dtype, void* workspace,
                size_t workspace_bytes, void* stream);

/* gx (N, Cin, *in) = gradient of the PADDED tile — torch.nn.grad.conv*_input as
 * called at jigsaw/modules/convolution/_conv/distributed.py:346-355. */
int jg_conv_dgrad(void* gx, const void* w, const void* g, const jg_conv_desc* desc,
                  int dtype, void* workspace, size_t workspace_bytes, void* stream);

/* Framed input. The halo-padded tile is mostly a shifted copy of the own tile, so the
 * framed entry points read the own tile x_tile (N, Cin, *geom->size) wherever a
 * kernel's window lies inside it, and the padded tensor x_frame (N, Cin, *desc->in_size,
 * geom->size + lo + hi = desc->in_size, planes = batch * c_in) only near the edges.
 * x_frame therefore only needs the frame that jg_halo_assemble_frame_3d writes with
 * the bands of jg_conv_frame_bands; results are bit-identical to jg_conv_fwd /
 * jg_conv_wgrad(_bias) on the fully assembled x_aug (the reference's halo_gather +
 * F.conv path, distributed.py:264-293, and conv*_weight, :359-368). gb may be NULL.
 * All three return JG_ERR_UNSUPPORTED where only the unframed kernels exist. */
int jg_conv_frame_bands(const jg_conv_desc* desc, const jg_halo_geom* geom, int dtype,
                        int32_t band_lo[3], int32_t band_hi[3]);
int jg_conv_fwd_framed(void* y, const void* x_frame, const void* x_tile, const void* w,
                       const void* bias, const jg_conv_desc* desc, const jg_halo_geom* geom,
                       int dtype, void* workspace, size_t workspace_bytes, void* stream);
int jg_conv_wgrad_framed(void* gw, void* gb, const void* x_frame, const void* x_tile,
                         const void* g, const jg_conv_desc* desc, const jg_halo_geom* geom,
                         int dtype, void* workspace, size_t workspace_bytes, void* stream);

/* jg_conv_dgrad with the first half of the fold fused into its epilogue
 * (distributed.py:346-355 followed by the sends of halo.py:222-226): `desc`
 * describes the convolution on the padded tile as for jg_conv_dgrad and `geom`
 * says where the own tile sits inside it (size + lo + hi = desc->in_size,
 * planes = batch * c_in). Cells of the padded gradient inside the tile go to gx
 * (planes, *size) as `0 + v`; halo cells go to send[slot of the neighbour that
 * owns them] in the layout of jg_halo_pack_3d(from_padded = 1); a NULL slot
 * drops them. Returns JG_ERR_UNSUPPORTED where only the unfused path exists
 * (workspace as for JG_CONV_DGRAD). Finish with jg_halo_fold_border_3d. */
int jg_conv_dgrad_fold(void* gx, void* const send[27], const void* w, const void* g,
                       const jg_conv_desc* desc, const jg_halo_geom* geom, int dtype,
                       void* workspace, size_t workspace_bytes, void* stream);

/* gw (Cout, Cin, *kernel) — torch.nn.grad.conv*_weight as called at
 * jigsaw/modules/convolution/_conv/distributed.py:359-368. Deterministic
 * (fixed-order two-stage reduction, no atomics). */
int jg_conv_wgrad(void* gw, const void* x, const void* g, const jg_conv_desc* desc,
                  int dtype, void* workspace, size_t workspace_bytes, void* stream);

/* jg_conv_wgrad that also produces gb (Cout,) = sum of g over batch and pixels
 * (_sum_grad_bias, jigsaw/modules/convolution/_conv/config.py:117-120) from the
 * same pass over g, saving the separate read of g by jg_bias_grad. Workspace as
 * for JG_CONV_WGRAD. Returns JG_ERR_UNSUPPORTED where only the separate kernels
 * cover the problem. */
int jg_conv_wgrad_bias(void* gw, void* gb, const void* x, const void* g,
                       const jg_conv_desc* desc, int dtype, void* workspace,
                       size_t workspace_bytes, void* stream);

/* gb (C,) = sum of g (N, C, spatial...) over batch and spatial axes —
 * _sum_grad_bias, jigsaw/modules/convolution/_conv/config.py:117-120.
 * `spatial` = product of the spatial extents. */
size_t jg_bias_grad_workspace_bytes(int64_t batch, int64_t channels, int64_t spatial);
int jg_bias_grad(void* gb, const void* g, int64_t batch, int64_t channels,
                 int64_t spatial, int dtype, void* workspace, size_t workspace_bytes,
                 void* stream);

/* ------------------------------------------------------------------------- *
 * Attention core of the ring step (MFMA kernels: bf16 at head sizes 64, 96, 128; fp16 at 96, 128)
 *
 * q (batch, sq, d), k / v (batch, sk, d), dense, `batch` = all leading axes
 * flattened (b*h for the "bhsd" layout of jigsaw's sdpa / math cores). One dtype
 * per call; softmax and accumulation in fp32. Non-causal, no dropout.
 * `bias` (optional, fp32): additive score bias / mask of shape
 * (bias_period, sq, sk); batch entry i uses bias[i % bias_period]
 * (windowed attention with a relative-position bias, examples/swin.py:146-151).
 * ------------------------------------------------------------------------- */

/* out = softmax(scale * q k^T + bias) v, lse = natural-log sum-exp of the scaled
 * scores, (batch, sq) fp32 — cores/math.forward
 * (jigsaw/modules/attention/_functional/cores/math.py:31-78) and the contract of
 * cores/__init__.py:1-15.
 * Fused ring merge: when out_acc (fp32, shape of out) and lse_acc (fp32,
 * (batch, sq)) are given, this chunk's result is merged into them in place,
 *   w = sigmoid(lse - lse_acc); out_acc += w*(out - out_acc); lse_acc = logaddexp,
 * which is _online_softmax_merge_ (forward.py:23-61) without the round trip of
 * out_j through HBM; `out` / `lse` may then be NULL (bf16 with d = 64, 96 or 128, fp16
 * with d = 96 or 128, sq and sk multiples of 128; fp32 with d = 32, 64 or 128, no bias,
 * 16-byte aligned tensors, any sq and sk; JG_ERR_UNSUPPORTED otherwise).
 * fp32 without a bias at d = 32, 64 or 128 runs on the fp32 matrix-core instructions
 * (forward and backward), other fp32 calls on one-thread-per-row kernels.
 * d must be one of 8, 16, 32, 64, 96, 128 (JG_ERR_UNSUPPORTED otherwise; zero
 * columns appended to q, k, v leave out's other columns and lse unchanged). */
int jg_attn_fwd(void* out, float* lse, const void* q, const void* k, const void* v,
                int64_t batch, int64_t sq, int64_t sk, int64_t d, float scale,
                const float* bias, int64_t bias_period, float* out_acc,
                float* lse_acc, int dtype, void* stream);

/* (dq, dk, dv) of one chunk from the GLOBAL out / lse of the ring
 * (cores/math.backward, cores/math.py:81-149): p = exp(scale*q k^T + bias - lse),
 * delta = rowsum(dout*out), ds = p*(dout v^T - delta)*scale, dq = ds k,
 * dk = ds^T q, dv = p^T dout. dq/dk/dv have the dtype of the inputs.
 * dbias (optional, fp32, (batch, sq, sk)) receives p*(dout v^T - delta), the
 * gradient of the additive bias per batch entry.
 * workspace: jg_attn_bwd_workspace_bytes(batch, sq, sk, d) bytes of scratch. */
size_t jg_attn_bwd_workspace_bytes(int64_t batch, int64_t sq, int64_t sk, int64_t d);
int jg_attn_bwd(void* dq, void* dk, void* dv, const void* dout, const void* q,
                const void* k, const void* v, const void* out, const float* lse,
                int64_t batch, int64_t sq, int64_t sk, int64_t d, float scale,
                const float* bias, int64_t bias_period, float* dbias, int dtype,
                void* workspace, size_t workspace_bytes, void* stream);

/* The backward loop of one rank's ring over n_chunks RESIDENT chunks in one call
 * (_functional/backward.py:176-277 with the chunks the forward saved: step s takes chunk s):
 * k[c], v[c] (batch, sk, d) are chunk c, dk[c], dv[c] receive this rank's partial for it (what
 * jg_attn_bwd returns for that chunk), dq the sum of the per-chunk dq, accumulated in fp32 and
 * rounded once (the reference adds the steps in q's dtype, backward.py:184, 269). k, v, dk, dv are
 * HOST arrays of n_chunks device pointers, read before the call returns. No bias.
 * Covered: bf16, d = 64, sq and sk multiples of 128, 1 <= n_chunks <= 16; JG_ERR_UNSUPPORTED
 * otherwise (call jg_attn_bwd per chunk and add the dq). workspace as for jg_attn_bwd. */
int jg_attn_bwd_chunks(void* dq, void* const* dk, void* const* dv, const void* dout, const void* q,
                       const void* const* k, const void* const* v, int64_t n_chunks, const void* out,
                       const float* lse, int64_t batch, int64_t sq, int64_t sk, int64_t d, float scale,
                       int dtype, void* workspace, size_t workspace_bytes, void* stream);

/* Windowed attention of a Swin block on the token grid itself (examples/swin.py:129-170:
 * F.scaled_dot_product_attention over (B, nW, heads, 64, 32) windows with attn_mask = the
 * relative-position bias, index of examples/swin.py:99-104, plus the shift mask of 107-126).
 * q, k, v, out: (images, heads, gh * gw, 32) bf16, tokens in row-major grid order; the kernel
 * addresses the 8 x 8 windows in place, so no window partition is materialised. table: (225, heads)
 * fp32, the learned bias by relative position. side: (windows of one image, 64) bytes or NULL, a
 * code per token; tokens of one window with different codes do not attend each other.
 * lse: (images * windows * heads, 64) fp32, for the backward. */
int jg_attn_swin_fwd(void* out, float* lse, const void* q, const void* k, const void* v, const float* table,
                     const uint8_t* side, int64_t images, int64_t heads, int64_t gh, int64_t gw, int64_t d,
                     float scale, int dtype, void* stream);

/* Gradients of jg_attn_swin_fwd (autograd of the same call in the reference). dtable: (225, heads)
 * fp32 or NULL; when wanted, workspace must hold jg_attn_swin_bwd_workspace_bytes bytes. */
size_t jg_attn_swin_bwd_workspace_bytes(int64_t images, int64_t heads, int64_t gh, int64_t gw);
int jg_attn_swin_bwd(void* dq, void* dk, void* dv, float* dtable, const void* dout, const void* q, const void* k,
                     const void* v, const void* out, const float* lse, const float* table, const uint8_t* side,
                     int64_t images, int64_t heads, int64_t gh, int64_t gw, int64_t d, float scale, int dtype,
                     void* workspace, size_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* JIGSAW_HIP_H */
