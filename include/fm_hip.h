/* C ABI of libfmhip.so: hand-written HIP kernels (gfx950 / MI355X) for ForgeMind's
 * packed-kernel hot path.
 *
 * Conventions shared by every entry point
 *   - plain pointers and sizes only; all tensor pointers are DEVICE pointers to
 *     row-major, densely packed data (row stride == row width);
 *   - the caller owns every buffer, including scratch ("workspace"); the library never
 *     allocates, frees, retains a pointer or synchronises, so each call is a pure enqueue on
 *     `stream` (a hipStream_t passed as void*; NULL = the default stream) and can be
 *     captured into a HIP graph;
 *   - the device that is current on the calling thread must own the buffers;
 *   - inputs are never written;
 *   - return value 0 (FM_OK) on success, otherwise an fm_status code; fm_last_error()
 *     returns a thread-local message for the last failure on the calling thread;
 *   - element types are selected with fm_dtype codes; math is fp32 with one rounding at
 *     the store, and every reduction runs in a fixed order (no float atomics), so results
 *     are bit-reproducible run to run.
 *
 * "Reference" below is xygamer179-boop/ForgeMinds; each entry point names the reference
 * interface (file:line) it stands in for.
 */
#ifndef FM_HIP_H_
#define FM_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* fm_stream_t; /* hipStream_t */

enum fm_dtype { FM_F32 = 0, FM_F16 = 1, FM_BF16 = 2 };

enum fm_status {
  FM_OK = 0,
  FM_ERR_INVALID = 1,     /* bad argument (null pointer, non-positive size, bad enum) */
  FM_ERR_UNSUPPORTED = 2, /* shape or dtype outside what the kernels handle */
  FM_ERR_LAUNCH = 3,      /* the HIP runtime rejected a launch */
  FM_ERR_WORKSPACE = 4    /* workspace pointer missing or too small */
};

enum fm_reduction { FM_REDUCE_NONE = 0, FM_REDUCE_SUM = 1, FM_REDUCE_MEAN = 2 };

/* ABI version (bumped on any signature change) and last error text. */
int fm_version(void);
const char* fm_last_error(void);

/* Name of the last main kernel (template arguments resolved, e.g.
 * "ce_bwd_kernel<bf16_t, 1024, 4>") that an entry point enqueued from the calling thread; empty
 * before the first launch. A measurement hook: the benchmark keys profiler byte counts by it, so
 * a figure can never be attached to a kernel that did not run. Not part of the reference surface. */
const char* fm_last_kernel(void);

/* Launch-shape parameters for another part or shape: "norm_fwd_blocks_per_cu" and
 * "norm_bwd_blocks_per_cu" (workgroups of the persistent norm grids per compute unit; the second
 * also sizes the backward's workspace, so ask fm_*_bwd_workspace again after changing it),
 * "vocab_threads" (256 / 512 / 1024) and "vocab_unroll" (2 / 4 / 8) for the kernels that give a
 * workgroup a whole vocabulary row. None selects between code paths and no result depends on
 * them. Process-wide. value <= 0 restores the built-in choice; unknown names return
 * FM_ERR_INVALID. Not part of the reference surface. */
int fm_set_param(const char* name, int value);

/* STREAM-style probe with the kernels' own access pattern (16-byte non-temporal accesses, one
 * 64 KiB chunk per workgroup): mode 0 reads `bytes` from src (sink: one uint32 on device, never
 * written for ordinary data), mode 1 copies src to dst. Used by bench.py to report the HBM
 * ceiling this GPU reaches and to calibrate profiler byte counters against a known transfer.
 * No counterpart in the reference. bytes must be a multiple of 16. */
int fm_stream_probe(const void* src, void* dst, uint32_t* sink, size_t bytes, int mode,
                    fm_stream_t stream);

/* The floor of a row kernel: `reads` (1-3) input streams a, b, c and `writes` (0-2) output streams
 * o1, o2 of `bytes` each are swept once with 16-byte accesses and no arithmetic beyond an xor
 * (read-only sweeps keep their loads alive through `sink`, one uint32 on the device that ordinary
 * data never reaches). Loads are non-temporal like the row kernels'; store_kind 0 = plain,
 * 1 = non-temporal, 2 = o1 plain and o2 non-temporal. A workgroup of `threads` threads moves tiles
 * of threads * vecs_per_thread vectors (256x1, 256x2, 256x4, 512x2, 512x4, 1024x1, 1024x4); `grid`
 * workgroups walk the tiles (<= 0: one workgroup per tile). bytes must be a whole number of tiles.
 * bench.py times it on each workload's own buffers, with that workload's read / write mix, and
 * reports the workload's step as a fraction of the best such sweep. No counterpart in the
 * reference. */
int fm_stream_probe_mix(const void* a, const void* b, const void* c, void* o1, void* o2,
                        uint32_t* sink, size_t bytes, int reads, int writes, int store_kind,
                        int threads, int vecs_per_thread, int64_t grid, fm_stream_t stream);

/* ------------------------------------------------------------------ RMSNorm
 * Replaces _launch_rms_fwd / _rms_layernorm_forward (forgemind/kernels/norm.py:1095-1101,
 * 133-175); semantics of _fallback.rms_norm (forgemind/kernels/_fallback.py:26-30):
 *   r = rsqrt(mean(x^2) + eps);  y = ((x * r) * w) rounded once to x's dtype;  rstd[i] = r.
 * x, y: [n, d] of x_dtype; w: [d] of w_dtype (x_dtype or FM_F32); rstd: [n] fp32. */
int fm_rmsnorm_fwd(const void* x, const void* w, void* y, float* rstd, int64_t n, int64_t d,
                   int x_dtype, int w_dtype, float eps, fm_stream_t stream);

/* Bytes of scratch fm_rmsnorm_bwd / fm_add_rmsnorm_bwd need for the fp32 partial weight
 * gradients (the reference's `[programs, n_cols]` buffer, norm.py:845-870, 1143-1146). */
size_t fm_rmsnorm_bwd_workspace(int64_t n, int64_t d, int x_dtype);

/* Replaces _launch_rms_bwd / _rms_layernorm_backward + _rms_sum_dw_partials
 * (norm.py:1104-1115, 179-231, 234-316, 571-593):
 *   xh = x * rstd; g = dy * w; dx = rstd * (g - xh * mean(g * xh));  dw = sum_rows dy * xh.
 * dx: [n, d] of x_dtype; dw: [d] of w_dtype (fp32 accumulation, fixed summation order).
 * dw may be NULL (frozen weight): then no workspace is needed. */
int fm_rmsnorm_bwd(const void* x, const void* w, const float* rstd, const void* dy, void* dx,
                   void* dw, void* workspace, size_t workspace_bytes, int64_t n, int64_t d,
                   int x_dtype, int w_dtype, fm_stream_t stream);

/* fm_rmsnorm_bwd for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc): the same kernels and the same results,
 * with the partial weight gradients in a buffer of FM_RMSNORM_BWD_STATIC_BYTES that is built
 * into the library (one copy per GPU, held until the process ends) instead of a workspace
 * argument. No counterpart in the reference. Allocates nothing; the first call on a device
 * looks the buffer's address up once (make that call before starting a capture). Shapes whose
 * partial rows need more than the buffer return FM_ERR_UNSUPPORTED: the condition is
 * fm_rmsnorm_bwd_workspace(n, d, x_dtype) <= FM_RMSNORM_BWD_STATIC_BYTES, i.e. (partial rows) x d
 * x 4 bytes with one partial row per workgroup of the persistent grid -- compute units x
 * "norm_bwd_blocks_per_cu" (1 unless changed with fm_set_param). On a 256-unit part with the
 * default that is every d <= 8192; with two workgroups per unit, d <= 4096. All calls on one
 * GPU share the buffer: calls that overlap in time on one GPU (two streams) race; calls on one
 * stream, or on different GPUs, do not. */
#define FM_RMSNORM_BWD_STATIC_BYTES ((size_t)8 << 20)
int fm_rmsnorm_bwd_static(const void* x, const void* w, const float* rstd, const void* dy, void* dx,
                          void* dw, int64_t n, int64_t d, int x_dtype, int w_dtype,
                          fm_stream_t stream);

/* Replaces _launch_addrms_fwd / _addrms_fwd (norm.py:1118-1131, 1001-1047) with the
 * rounding points of _fallback.add_rms_norm (_fallback.py:33-35):
 *   xn = x + delta rounded to x's dtype; y = rms_norm(xn, w, eps) computed from the rounded xn. */
int fm_add_rmsnorm_fwd(const void* x, const void* delta, const void* w, void* xn, void* y,
                       float* rstd, int64_t n, int64_t d, int x_dtype, int w_dtype, float eps,
                       fm_stream_t stream);

/* Replaces _launch_addrms_bwd / _addrms_bwd (norm.py:1134-1148, 1050-1086):
 *   dx = rstd * (gy*w - xh * mean(gy*w*xh)) + gxn;  ddelta == dx;  dw = sum_rows gy * xh.
 * gxn (gradient of the residual output) may be NULL (treated as zero). ddelta may be NULL or
 * equal to dx (the two gradients are the same values; a second buffer is only written when
 * a distinct pointer is given). dw may be NULL. */
int fm_add_rmsnorm_bwd(const void* xn, const void* w, const float* rstd, const void* gy,
                       const void* gxn, void* dx, void* ddelta, void* dw, void* workspace,
                       size_t workspace_bytes, int64_t n, int64_t d, int x_dtype, int w_dtype,
                       fm_stream_t stream);

/* ------------------------------------------------------------------ LayerNorm
 * No kernel of this name exists in the reference (its norm kernels are the RMS pair,
 * kernels/norm.py:133-316); these follow the same contract and rounding rule as the RMSNorm
 * entry points above (_fallback.py:15-35: fp32 math on the stored values, one rounding) with
 * torch.nn.functional.layer_norm's arithmetic:
 *   mean = sum(x)/d;  rstd = rsqrt(sum((x-mean)^2)/d + eps);  y = ((x-mean)*rstd)*w + bias.
 * bias may be NULL. mean, rstd: [n] fp32, kept for the backward. */
int fm_layernorm_fwd(const void* x, const void* w, const void* bias, void* y, float* mean,
                     float* rstd, int64_t n, int64_t d, int x_dtype, int w_dtype, float eps,
                     fm_stream_t stream);

/* xn = x + delta rounded to x's dtype; y = layer_norm(xn) computed from the rounded xn
 * (the residual-add form of fm_add_rmsnorm_fwd). */
int fm_add_layernorm_fwd(const void* x, const void* delta, const void* w, const void* bias,
                         void* xn, void* y, float* mean, float* rstd, int64_t n, int64_t d,
                         int x_dtype, int w_dtype, float eps, fm_stream_t stream);

/* Bytes of scratch fm_layernorm_bwd needs (fp32 partial rows for dw and db). */
size_t fm_layernorm_bwd_workspace(int64_t n, int64_t d, int x_dtype);

/* g = dy*w; xh = (x-mean)*rstd; dx = rstd * ((g - mean(g)) - xh*mean(g*xh)) [+ gxn];
 * dw = sum_rows dy*xh; db = sum_rows dy. x is the normalised input (xn of the add form);
 * gxn (gradient of the residual output of the add form) may be NULL; dw and db may be NULL
 * (no workspace is needed when both are). */
int fm_layernorm_bwd(const void* x, const void* w, const float* mean, const float* rstd,
                     const void* dy, const void* gxn, void* dx, void* dw, void* db,
                     void* workspace, size_t workspace_bytes, int64_t n, int64_t d, int x_dtype,
                     int w_dtype, fm_stream_t stream);

/* ------------------------------------------------------------------ cross entropy
 * Replaces the F.cross_entropy(reduction="sum") / n reduction of logits_cross_entropy and
 * chunked_cross_entropy (forgemind/loss.py:54-70, 23-51):
 *   row_loss[i] = logsumexp(logits[i,:]) - logits[i, labels[i]]   (0 where labels[i] == ignore_index)
 *   n_valid = max(1, #{labels != ignore_index})
 *   loss = sum(row_loss) / n_valid for FM_REDUCE_MEAN (loss.py:63-70),
 *          sum(row_loss) for FM_REDUCE_SUM (one chunk of loss.py:36-38)
 * logits: [n, v] of dtype; labels: [n] int64; lse, row_loss: [n] fp32 (lse is what the
 * backward re-uses instead of a stored softmax); loss, n_valid: fp32 scalars on device.
 * One read of logits. n == 0 yields loss 0 and n_valid 1.
 * lse may be NULL when no backward will follow (evaluation): the logits are then streamed past
 * the caches throughout. With lse the last 256 MiB of them (what the part's memory-side cache
 * holds) are read with cached loads, and fm_ce_bwd, called next, finds those rows there. */
int fm_ce_fwd(const void* logits, const int64_t* labels, float* lse, float* row_loss,
              float* loss, float* n_valid, int64_t n, int64_t v, int dtype,
              int64_t ignore_index, int reduction, fm_stream_t stream);

/* Backward of the above (what autograd derives for loss.py:65-70):
 *   dlogits[i,j] = (exp(logits[i,j] - lse[i]) - [j == labels[i]]) * grad_out / n_valid
 * for rows with a valid label, 0 for ignored rows (those rows are not read).
 * grad_out: device fp32 scalar, or NULL for 1. n_valid: the scalar fm_ce_fwd wrote, or NULL
 * for 1 (the gradient of the FM_REDUCE_SUM loss). dlogits: [n, v] of dtype. */
int fm_ce_bwd(const void* logits, const int64_t* labels, const float* lse, const float* n_valid,
              const float* grad_out, void* dlogits, int64_t n, int64_t v, int dtype,
              int64_t ignore_index, fm_stream_t stream);

/* Loss AND gradient of loss.py:54-70 from one read of the logits: fm_ce_fwd's outputs plus
 *   dlogits[i,j] = (softmax(logits[i,:])[j] - [j == labels[i]]) / n_valid   (FM_REDUCE_MEAN)
 * i.e. fm_ce_bwd with grad_out = 1, written in the same pass (a training step whose loss is
 * the last node has exactly that upstream gradient; fm_scale_inplace applies any other one).
 * Rows stay in registers between the log-sum-exp and the store, so the step moves 2 + 2
 * bytes per 16-bit logit instead of 2 + 2 + 2. dlogits may be the logits buffer itself
 * (the way the reference's KL writes its gradient into an owned student tensor,
 * kernels/kl.py:146-150, 157-160); lse may be NULL. Rows wider than 128 KiB stay on the chip
 * all the same (registers and LDS of one workgroup per compute unit hold 384 KiB; what a row has
 * beyond that, up to twice that width, is streamed and read again); wider rows still and unaligned
 * buffers are swept twice inside the same launch (faster than two launches, not single-read).
 * lse of ignored rows is written as 0 (those rows are not read). */
int fm_ce_loss_grad(const void* logits, const int64_t* labels, float* lse, float* row_loss,
                    float* loss, float* n_valid, void* dlogits, int64_t n, int64_t v, int dtype,
                    int64_t ignore_index, int reduction, fm_stream_t stream);

/* x[i] *= *factor for count elements of dtype, in place; a factor of exactly 1 returns
 * without touching x. Stands in for `grad * g` in the backward of a loss whose gradient was
 * produced in the forward (kernels/kl.py:181-191 does that multiply unconditionally). */
int fm_scale_inplace(void* x, const float* factor, int64_t count, int dtype, fm_stream_t stream);

/* ------------------------------------------------------------------ distillation KL
 * Replaces _kl_fwd_bwd_kernel's loss half (forgemind/kernels/kl.py:73-135, 143-179);
 * semantics of _fallback.kl_div_logits (_fallback.py:52-69) on logits scaled by
 * inv_temperature:  row_kl[i] = sum_j p_t (log p_t - log p_s),  p = softmax(logits * inv_temperature).
 * One pass over both rows (online max / sum-exp); lse_s, lse_t ([n] fp32, of the scaled
 * logits) are saved for the backward. loss (device fp32 scalar, may be NULL) receives
 * sum(row_kl) for FM_REDUCE_SUM, sum/n for FM_REDUCE_MEAN and is left untouched for
 * FM_REDUCE_NONE. */
int fm_kl_fwd(const void* student, const void* teacher, float* lse_s, float* lse_t,
              float* row_kl, float* loss, int64_t n, int64_t v, int dtype,
              float inv_temperature, int reduction, fm_stream_t stream);

/* KL AND its gradient from one read of both rows, the dataflow of the reference's kernel
 * (kl.py:73-135 writes dKL/dstudent in the forward, _KLDivFn.forward kl.py:154-176):
 * fm_kl_fwd's outputs plus dstudent = fm_kl_bwd's result for grad_out = 1 and
 * scale = 1/n (FM_REDUCE_MEAN) or 1 (FM_REDUCE_SUM). Rows of at most 32 KiB stay in
 * registers between the log-sum-exps and the store (4 + 2 bytes per pair of 16-bit logits
 * instead of 4 + 4 + 2); rows of up to 512 KiB are kept in the registers and LDS of one workgroup
 * per compute unit (496 KiB of each row pair; the rest is read twice) while that workgroup already
 * loads its next row; wider rows and unaligned buffers are swept twice inside the same launch.
 * dstudent may be the student buffer itself when
 * grad_dtype == dtype (kl.py:146-150, reuse=True); lse_s / lse_t may be NULL.
 * fm_scale_inplace applies an upstream gradient other than 1. */
int fm_kl_loss_grad(const void* student, const void* teacher, float* lse_s, float* lse_t,
                    float* row_kl, float* loss, void* dstudent, int64_t n, int64_t v, int dtype,
                    int grad_dtype, float inv_temperature, int reduction, fm_stream_t stream);

/* fm_kl_fwd that also returns the exact top-k of every teacher row from the same pass over
 * the logits. The reference has no fused form: a distillation step calls kl_div_logits
 * (kernels/kl.py:194-232) and topk (kernels/topk.py:273-297) one after the other, reading the
 * teacher twice. Selection follows topk.py:13-19 on the raw teacher logits (softmax and a
 * positive temperature keep the order): topk_values [n, k] (row dtype, may be NULL),
 * topk_indices [n, k] (int32 or int64 by index_bits), topk_probs [n, k] fp32 (may be NULL) =
 * softmax(teacher * inv_temperature) at the selected columns. Rows wider than 1040 KiB or
 * k > 512 return FM_ERR_UNSUPPORTED; the caller then uses fm_kl_fwd + fm_topk. */
int fm_kl_fwd_topk(const void* student, const void* teacher, float* lse_s, float* lse_t,
                   float* row_kl, float* loss, void* topk_values, void* topk_indices,
                   float* topk_probs, int64_t n, int64_t v, int k, int dtype, int index_bits,
                   float inv_temperature, int reduction, fm_stream_t stream);

/* fm_kl_fwd_topk that also writes the gradient of the student in the same launch (a second
 * sweep of the row after the selection): dstudent [n, v] of
 * dtype = fm_kl_bwd's result for grad_out = 1 and scale = 1/n (FM_REDUCE_MEAN) or 1
 * (FM_REDUCE_SUM), a buffer of its own. One launch for a whole distillation step (KL, its
 * gradient, the teacher's top-k). No counterpart in the reference (see fm_kl_fwd_topk). */
int fm_kl_loss_grad_topk(const void* student, const void* teacher, float* lse_s, float* lse_t,
                         float* row_kl, float* loss, void* dstudent, void* topk_values,
                         void* topk_indices, float* topk_probs, int64_t n, int64_t v, int k, int dtype,
                         int index_bits, float inv_temperature, int reduction, fm_stream_t stream);

/* Gradient wrt the (unscaled) student logits, recomputed from the saved lse values
 * (the reference stores it from the forward, kl.py:112-134, and rescales it in
 * _KLDivFn.backward, kl.py:181-191):
 *   dstudent[i,j] = (p_s - p_t) * inv_temperature * scale * g_i
 * g_i = grad_out[i] when grad_per_row != 0, grad_out[0] otherwise, 1 when grad_out is NULL;
 * `scale` carries the 1/n of the mean reduction. dstudent: [n, v] of grad_dtype. */
int fm_kl_bwd(const void* student, const void* teacher, const float* lse_s, const float* lse_t,
              const float* grad_out, int grad_per_row, void* dstudent, int64_t n, int64_t v,
              int dtype, int grad_dtype, float inv_temperature, float scale, fm_stream_t stream);

/* ------------------------------------------------------------------ top-k
 * Replaces _fused / _topk_threshold_kernel + _topk_select_kernel
 * (forgemind/kernels/topk.py:234-251, 59-218). Exact top-k over the last dim in the canonical
 * order of topk.py:13-16: value descending, index ascending inside ties, smallest indices
 * win at the k-th value; NaN counts as the largest value and is passed through.
 * x: [n, v] of dtype; values: [n, k] of dtype (may be NULL); indices: [n, k] int32 when
 * index_bits == 32, int64 when index_bits == 64. 1 <= k <= min(v, 512). */
int fm_topk(const void* x, void* values, void* indices, int64_t n, int64_t v, int k, int dtype,
            int index_bits, fm_stream_t stream);

/* ------------------------------------------------------------------ softmax (last dim)
 * Replaces _softmax_kernel (forgemind/kernels/softmax.py:27-80): y = exp(x - max) / sum. */
int fm_softmax_fwd(const void* x, void* y, int64_t n, int64_t v, int dtype, fm_stream_t stream);

/* Replaces the tensor expression of _Softmax.backward (forgemind/kernels/softmax.py:108-115):
 * dx = (dy - sum(dy * y)) * y per row, fp32 math on the stored y and dy, one rounding.
 * y, dy, dx: [n, v] of dtype, three distinct buffers. */
int fm_softmax_bwd(const void* y, const void* dy, void* dx, int64_t n, int64_t v, int dtype,
                   fm_stream_t stream);

/* ------------------------------------------------------------------ MoE router + dispatch permutation
 * Replaces the aten sequence of Router.forward and MoE.forward
 * (forgemind/moe.py:86-91, 52-60, 232-236): probs = softmax(logits) in fp32; top-k of probs
 * in the canonical order above (lowest expert index wins ties); weights renormalised to sum
 * to 1; per-expert counts; and the stable sort of the flat assignments by expert:
 *   flat[p] = idx[p / k][p % k];  slot[p] = position of p after the stable sort;
 *   order[slot[p]] = p  (== torch.sort(flat, stable=True).indices).
 * logits: [n, e] of dtype (fp32 math inside); idx: [n, k] int32; weights: [n, k] fp32;
 * counts: [e] int32; slot, order: [n*k] int32 (either may be NULL: then only routing and
 * counts are produced when both are NULL). stats: fp32 [e+3] or NULL; receives the auxiliary
 * losses of moe.py:92-95 and the sums behind them, without another pass over the logits:
 *   stats[j] = sum_rows probs[:, j] (j < e),  stats[e] = sum_rows logsumexp(logits)^2,
 *   stats[e+1] = aux = E * sum_j counts[j] / (n k) * stats[j] / n,  stats[e+2] = z = stats[e] / n,
 * summed in a fixed order. 1 <= k <= 16, k <= e <= 512, n*k < 2^31.
 * Probabilities below the smallest normal fp32 (a logit more than 87 below the row maximum) come
 * out as zero and tie by expert index; a row holding a NaN or +inf, or only -inf, has NaN
 * probabilities throughout, selects experts 0..k-1 and gets NaN weights. */
size_t fm_route_workspace(int64_t n, int e, int k);
int fm_route(const void* logits, int32_t* idx, float* weights, int32_t* counts, int32_t* slot,
             int32_t* order, float* stats, void* workspace, size_t workspace_bytes, int64_t n,
             int e, int k, int dtype, fm_stream_t stream);

/* Gradient of fm_route's differentiable outputs wrt the logits, in one pass. Replaces what
 * autograd derives from Router.forward (forgemind/moe.py:86-95): through the renormalised top-k
 * weights (gweights: fp32 [n, k] gradient of `weights`, or NULL), through the load-balance loss
 * aux = E * sum_e frac_e * mean_rows(probs)_e with frac = counts / (n k) held constant
 * (moe.py:92-94; g_aux: fp32 device scalar or NULL, needs counts), and through the z-loss
 * mean_rows(logsumexp^2) (moe.py:95; g_z: fp32 device scalar or NULL). idx, counts: as written
 * by fm_route. dlogits: [n, e] of dtype. Same limits as fm_route. */
int fm_route_bwd(const void* logits, const int32_t* idx, const float* gweights, const int32_t* counts,
                 const float* g_aux, const float* g_z, void* dlogits, int64_t n, int e, int k, int dtype,
                 fm_stream_t stream);

/* ------------------------------------------------------------------ token moves around the permutation
 * Replaces `xs = x[order // k]` (forgemind/moe.py:234-235): xs[s, :] = scale * x[order[s] / k, :]
 * with scale = scale_flat[order[s]] when scale_flat (fp32 [n*k], indexed by flat assignment)
 * is given, 1 otherwise. x: [n, d]; xs: [n*k, d]; order: [n*k] int32 from fm_route.
 * With a scale it is also the backward of fm_moe_combine wrt ys (x = dout, scale = weights).
 * 1 <= k <= 16 for all four token moves (fm_route's range). */
int fm_moe_gather(const void* x, const int32_t* order, const float* scale_flat, void* xs, int64_t n,
                  int64_t d, int k, int dtype, fm_stream_t stream);

/* fm_moe_gather from the token's side, for callers that hold `slot` (the inverse of `order`, also
 * written by fm_route): xs[slot[t*k + j], :] = scale * x[t, :] for j < k, scale = scale_flat[t*k + j]
 * or 1. The same xs, bit for bit; a token row is read once instead of k times. */
int fm_moe_scatter(const void* x, const int32_t* slot, const float* scale_flat, void* xs, int64_t n,
                   int64_t d, int k, int dtype, fm_stream_t stream);

/* Replaces `ys * w[order]` + `zeros.index_add_(0, order // k, ys)` (moe.py:247-248) by a gather
 * per token through the slot array of fm_route:
 *   out[t, :] = sum_j weights[t, j] * ys[slot[t*k + j], :]   (fp32 sum in j order, one rounding)
 * weights: fp32 [n, k] or NULL for unit weights (then it is the backward of fm_moe_gather).
 * ys: [n*k, d]; out: [n, d]. No atomics: every output row is written once, deterministically. */
int fm_moe_combine(const void* ys, const float* weights, const int32_t* slot, void* out, int64_t n,
                   int64_t d, int k, int dtype, fm_stream_t stream);

/* Backward of fm_moe_combine wrt the weights: dweights[t, j] = <ys[slot[t*k+j], :], dout[t, :]>. */
int fm_moe_combine_dw(const void* ys, const void* dout, const int32_t* slot, float* dweights,
                      int64_t n, int64_t d, int k, int dtype, fm_stream_t stream);

/* ------------------------------------------------------------------ SwiGLU epilogues
 * Replace _swiglu_fwd_kernel / _swiglu_bwd_kernel and the split variants
 * (forgemind/kernels/swiglu.py:48-120); semantics of _fallback.swiglu (_fallback.py:48-49):
 * y = silu(gate) * up in fp32, one rounding. n counts elements; the split form reads a fused
 * projection x [rows, 2h] (gate = x[:, :h], up = x[:, h:]) and writes y [rows, h] / dx [rows, 2h]. */
int fm_swiglu_fwd(const void* gate, const void* up, void* y, int64_t n, int dtype, fm_stream_t stream);
int fm_swiglu_bwd(const void* gate, const void* up, const void* dy, void* dgate, void* dup, int64_t n,
                  int dtype, fm_stream_t stream);
int fm_swiglu_split_fwd(const void* x, void* y, int64_t rows, int64_t h, int dtype, fm_stream_t stream);
int fm_swiglu_split_bwd(const void* x, const void* dy, void* dx, int64_t rows, int64_t h, int dtype,
                        fm_stream_t stream);

/* ------------------------------------------------------------------ per-head RMSNorm + RoPE
 * Replace _qknorm_rope_fwd / _qknorm_rope_bwd (forgemind/kernels/rope.py:46-120); semantics of
 * _fallback.qk_norm_rope (_fallback.py:38-45). x, out, dout, dx: [b, t, h, d] of x_dtype (d even,
 * <= 512); w: [d] of w_dtype; cos, sin: fp32 [t, d/2]; rstd: fp32 [b*t*h]. dw ([d], w_dtype)
 * may be NULL; otherwise workspace of fm_qk_norm_rope_bwd_workspace bytes is needed. */
int fm_qk_norm_rope_fwd(const void* x, const void* w, const float* cosv, const float* sinv, void* out,
                        float* rstd, int64_t b, int64_t t, int64_t h, int64_t d, int x_dtype, int w_dtype,
                        float eps, fm_stream_t stream);
size_t fm_qk_norm_rope_bwd_workspace(int64_t b, int64_t t, int64_t h, int64_t d);
int fm_qk_norm_rope_bwd(const void* x, const void* w, const float* cosv, const float* sinv,
                        const float* rstd, const void* dout, void* dx, void* dw, void* workspace,
                        size_t workspace_bytes, int64_t b, int64_t t, int64_t h, int64_t d, int x_dtype,
                        int w_dtype, fm_stream_t stream);

#ifdef __cplusplus
}
#endif

#endif /* FM_HIP_H_ */
