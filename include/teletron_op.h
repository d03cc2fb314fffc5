/*
 * teletron_op.h — C ABI of the MI355X (gfx950) fused normalisation kernels.
 *
 * This is the drop-in boundary for TeleTron's `teletron_op` native ops.  Every
 * entry point takes plain device pointers, sizes and a HIP stream handle; no
 * torch types appear in any signature.  All tensors are row-major and
 * contiguous: `rows x cols` bf16 for activations, bf16 for parameters, fp32 for
 * per-row statistics and for parameter gradients.
 *
 * Fast path: cols % 8 == 0 and every tensor 16-byte aligned (128-bit vector kernels).
 * tt_adaln_forward/backward, tt_rmsnorm_forward/backward and the tt_launch_*_forward entry
 * points also accept any other cols <= TT_MAX_COLS and 2-byte aligned tensors through
 * element-wise kernels (a correctness path, several times slower); the two-step backward
 * and the tt_launch_*_backward entry points return TT_ERR_UNSUPPORTED there.
 *
 * Two groups of entry points:
 *
 *  1. The native contract (tt_adaln_*, tt_rmsnorm_*): backward consumes the
 *     forward *input* x and recomputes the row statistics, so nothing but x has
 *     to be saved; parameter gradients are fp32 and may be per-sample
 *     ([n_batches, cols], n_batches = rows / rows_per_batch).
 *  2. The reference-compatible contract (tt_launch_*): argument for argument the
 *     launchers that the reference's pybind glue calls, including the saved
 *     x_norm / y tensors and bf16 parameter gradients.
 *
 * Return value: 0 (TT_OK) on success, otherwise one of the TT_ERR_* codes;
 * tt_error_string() maps a code to text and tt_last_hip_error() returns the
 * hipError_t recorded by the calling thread's last TT_ERR_HIP.  Kernels are
 * enqueued on `stream` (NULL = the default stream) of the *current* device and
 * the calls do not synchronise.  Apart from tt_adaln_backward_static (which says so) the
 * library keeps no mutable device state, so calls from several host threads on different
 * streams are safe.
 */
#ifndef TELETRON_OP_H_
#define TELETRON_OP_H_

#include <stddef.h>
#include <stdint.h>

#if defined(__GNUC__)
#define TT_API __attribute__((visibility("default")))
#else
#define TT_API
#endif

#ifdef __cplusplus
extern "C" {
#endif

#define TT_OK 0
#define TT_ERR_INVALID_ARGUMENT 1  /* null pointer, non-positive size, rows % rows_per_batch != 0 */
#define TT_ERR_UNSUPPORTED 2       /* shape outside what the entry point covers (see above; cols > TT_MAX_COLS) */
#define TT_ERR_WORKSPACE 3         /* workspace pointer null or smaller than *_workspace_bytes() */
#define TT_ERR_HIP 4               /* a HIP runtime call or kernel launch failed */
#define TT_ERR_STATIC_LIMIT 5      /* tt_adaln_backward_static: the shape needs more than TT_STATIC_WORKSPACE_BYTES */

#define TT_MAX_COLS 32768

/* Library version: major * 10000 + minor * 100 + patch. */
TT_API int tt_version(void);
TT_API const char* tt_error_string(int code);
TT_API int tt_last_hip_error(void);

/* ------------------------------------------------------------------ fused AdaLN
 * y = LayerNorm_noaffine(x) * (1 + scale) + shift
 *
 * Replaces launch_adaln_forward (teletron_op/fused_adaln/include/adaln_kernel.h:20-29,
 * teletron_op/fused_adaln/adaln_forward.cu:198-220) for any `cols`, with
 * per-sample modulation: scale/shift are [n_batches, cols] bf16 where row r uses
 * batch r / rows_per_batch (pass rows_per_batch = rows for a single [cols] vector,
 * the reference's only mode, adaln_forward.cu:171-172).  Unlike the reference it
 * does not emit x_norm; `mean` and `rstd` ([rows] fp32) are optional (NULL to skip).
 */
TT_API int tt_adaln_forward(void* y, const void* x, const void* scale, const void* shift,
                     float* mean, float* rstd,
                     int64_t rows, int64_t cols, int64_t rows_per_batch,
                     float eps, void* stream);

/* Backward of the above.  Replaces launch_adaln_backward + launch_adaln_scale_shift_backward
 * (adaln_kernel.h:31-44, adaln_backward.cu:129-151, scale_shift_backward.cu:129-147):
 *   g = dy * (1 + scale);  dx = rstd * (g - mean(g) - x_hat * mean(g * x_hat))
 *   dscale[b, c] = sum_{rows of batch b} dy * x_hat;  dshift[b, c] = sum dy
 * Inputs dy, x: [rows, cols] bf16; scale: [n_batches, cols] bf16.
 * Outputs dx: [rows, cols] bf16; dscale, dshift: [n_batches, cols] fp32.
 * `workspace` holds the per-workgroup partial column sums; it must be at least
 * tt_adaln_backward_workspace_bytes() (for the same shape, on the same device) and 16-byte
 * aligned; about 10 MB at rows 75600, cols 5120.  (With cols % 8 == 0 but a
 * misaligned tensor the element-wise path needs rows * 8 bytes instead, which can exceed
 * that figure for very short rows; TT_ERR_WORKSPACE is returned if it does not fit.)  The result is
 * bitwise reproducible run to run (fixed summation order, no atomics).
 */
TT_API int tt_adaln_backward(void* dx, float* dscale, float* dshift,
                      const void* dy, const void* x, const void* scale,
                      void* workspace, size_t workspace_bytes,
                      int64_t rows, int64_t cols, int64_t rows_per_batch,
                      float eps, void* stream);
TT_API size_t tt_adaln_backward_workspace_bytes(int64_t rows, int64_t cols, int64_t rows_per_batch);

/* tt_adaln_backward for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc): same arguments without the
 * workspace, same kernels, same results bit for bit.  No counterpart in the reference.  The
 * scratch memory (partial column sums) is a device array inside the library,
 * TT_STATIC_WORKSPACE_BYTES (16 MiB); every GPU on which the library's code is loaded holds its
 * own copy until the process ends, whether or not this entry point is ever called.  The call
 * performs no hipMalloc / hipFree.  The first call on a GPU looks up that GPU's address of the
 * array (hipGetSymbolAddress) and the launch plan's device properties; a call with rows == 0 does
 * only that and touches no pointer, for callers that want this set-up done at a chosen moment.
 * A shape that needs more scratch than the array holds is refused with TT_ERR_STATIC_LIMIT: the
 * need is what tt_adaln_backward_workspace_bytes() returns (10.2 MB at rows 75600, cols 5120), or
 * rows * 8 bytes when cols is not a multiple of 8 or a tensor is not 16-byte aligned.  All calls
 * on one GPU share the array: two calls that overlap in time on the same GPU (different streams
 * or host threads, or two replays of graphs that captured it) race and give wrong dscale /
 * dshift; calls that follow each other on one stream are safe (nothing in the array has to
 * start at zero).
 */
#define TT_STATIC_WORKSPACE_BYTES (16u << 20)
TT_API int tt_adaln_backward_static(void* dx, float* dscale, float* dshift,
                             const void* dy, const void* x, const void* scale,
                             int64_t rows, int64_t cols, int64_t rows_per_batch,
                             float eps, void* stream);

/* ------------------------------------------------------------------ fused RMSNorm
 * y = x * rsqrt(mean(x^2) + eps) * weight
 *
 * Replaces launch_rms_forward (teletron_op/fused_rmsnorm/include/rmsnorm_kernel.h:5-12,
 * teletron_op/fused_rmsnorm/rms_forward.cu:102-121) for any `cols` (the reference
 * covers cols == 128 only).  `rstd` ([rows] fp32) is optional.
 */
TT_API int tt_rmsnorm_forward(void* y, const void* x, const void* weight, float* rstd,
                       int64_t rows, int64_t cols, float eps, void* stream);

/* Backward: replaces launch_rms_backward + launch_rms_weight_backward
 * (rmsnorm_kernel.h:14-25, rms_backward.cu:91-112, weight_backward.cu:212-260):
 *   g = dy * weight;  dx = rstd * (g - x_hat * mean(g * x_hat));  dweight[c] = sum_rows dy * x_hat
 * Consumes x (not the forward output) and never divides by weight.
 * dweight: [cols] fp32.  Workspace as for tt_adaln_backward.
 */
TT_API int tt_rmsnorm_backward(void* dx, float* dweight,
                        const void* dy, const void* x, const void* weight,
                        void* workspace, size_t workspace_bytes,
                        int64_t rows, int64_t cols, float eps, void* stream);
TT_API size_t tt_rmsnorm_backward_workspace_bytes(int64_t rows, int64_t cols);

/* ------------------------------------------------------------------ two-step backward
 * The backward entry points above are these two steps back to back.  They are
 * exported so that a caller can time the streaming kernel on its own, or sum the
 * per-workgroup partials of several devices before the final reduction.
 * (No counterpart in the reference, whose column reductions are separate kernels
 * that re-read dout and x_norm: scale_shift_backward.cu:49-126, weight_backward.cu:59-145.)
 *
 * Step 1 writes dx and, into `workspace`, partial column sums laid out as
 * [n_batches][*n_partials][n_acc][cols] fp32 with n_acc = 2 (dscale, dshift) for
 * AdaLN and 1 for RMSNorm.  Step 2 reduces over the n_partials axis in a fixed order.
 */
TT_API int tt_adaln_backward_partials(void* dx, const void* dy, const void* x, const void* scale,
                               void* workspace, size_t workspace_bytes, int* n_partials,
                               int64_t rows, int64_t cols, int64_t rows_per_batch,
                               float eps, void* stream);
TT_API int tt_rmsnorm_backward_partials(void* dx, const void* dy, const void* x, const void* weight,
                                 void* workspace, size_t workspace_bytes, int* n_partials,
                                 int64_t rows, int64_t cols, float eps, void* stream);
/* out0 / out1: [n_batches, cols] fp32; out1 is NULL when n_acc == 1. */
TT_API int tt_reduce_partials(float* out0, float* out1, const void* workspace,
                       int n_batches, int n_partials, int n_acc, int64_t cols, void* stream);

/* ------------------------------------------------------------------ RMSNorm + rotary embedding
 * The QK-norm of Wan self-attention is followed at once by the rotary position embedding
 * (norm_q / norm_k then rope_apply: teletron/models/wan/wan_model.py:105-110,154-158), which
 * the reference runs as separate float64 complex torch ops.  These entry points do both in the
 * one pass over the tensor:
 *   t = x * rsqrt(mean(x^2) + eps) * weight                         (full hidden dimension)
 *   (y[2i], y[2i+1]) = (t[2i] + i t[2i+1]) * (cos + i sin)          per head, pair by pair
 * freqs is fp32 [seq_len][head_dim / 2][2] = (cos, sin) for position and complex index inside a
 * head (the reference's complex freqs[s, 1, head_dim / 2] viewed as real); row r uses position
 * r % seq_len, every head of a row the same table.  Backward multiplies dy by the conjugate and
 * continues as tt_rmsnorm_backward.  Requires cols % head_dim == 0, head_dim % 8 == 0, head_dim <= 256,
 * cols > 256, 16-byte aligned tensors (TT_ERR_UNSUPPORTED otherwise).  Workspace as for
 * tt_rmsnorm_backward.  No counterpart in teletron_op.
 */
TT_API int tt_rmsnorm_rope_forward(void* y, const void* x, const void* weight, const float* freqs, float* rstd,
                                   int64_t rows, int64_t cols, int64_t head_dim, int64_t seq_len,
                                   float eps, void* stream);
TT_API int tt_rmsnorm_rope_backward(void* dx, float* dweight, const void* dy, const void* x, const void* weight,
                                    const float* freqs, void* workspace, size_t workspace_bytes,
                                    int64_t rows, int64_t cols, int64_t head_dim, int64_t seq_len,
                                    float eps, void* stream);

/* Per-head variant: HunyuanVideo normalises every head on its own (head_dim = 128, one weight
 * vector shared by the heads) and applies the rotary embedding right after
 * (teletron/models/hunyuan/model.py:92-125).  x is [rows, head_dim] in memory order
 * [batch, token, head, head_dim], i.e. `heads` consecutive rows belong to one token; row r uses
 * position (r / heads) % seq_len.  freqs as above: (cos, sin) per position and pair
 * (diffusers' real cos / sin tables [seq_len, head_dim] hold each value twice: take every second
 * column).  Tokens that take no rotation (the text tokens appended in the single-stream blocks,
 * model.py:101-121) get (1, 0) entries.  head_dim % 8 == 0, head_dim <= 256, rows % heads == 0.
 * Workspace: tt_rmsnorm_backward_workspace_bytes(rows, head_dim). */
TT_API int tt_rmsnorm_rope_heads_forward(void* y, const void* x, const void* weight, const float* freqs, float* rstd,
                                         int64_t rows, int64_t head_dim, int64_t heads, int64_t seq_len,
                                         float eps, void* stream);
TT_API int tt_rmsnorm_rope_heads_backward(void* dx, float* dweight, const void* dy, const void* x, const void* weight,
                                          const float* freqs, void* workspace, size_t workspace_bytes,
                                          int64_t rows, int64_t head_dim, int64_t heads, int64_t seq_len,
                                          float eps, void* stream);

/* ------------------------------------------------------------------ gated residual add
 * out = x + gate * residual, the op that follows each fused AdaLN site in a DiT block;
 * gate is [n_batches, cols] bf16, broadcast over the rows of its batch.  teletron_op has no
 * kernel for it: the reference runs it as eager torch ops in GateModule.forward
 * (teletron/models/wan/wan_model.py:205-210) / GateWithGradReduce
 * (teletron/core/context_parallel/layers.py:24-36), whose arithmetic this replaces:
 *   forward   out = x + gate * residual
 *   backward  dresidual = dout * gate;  dgate[b, c] = sum_{rows of batch b} dout * residual
 *             (dx = dout: no kernel, the caller aliases it)
 * Vector path only (cols % 8 == 0, 16-byte aligned tensors).  dgate is fp32 [n_batches, cols],
 * reduced in a fixed order like the other parameter gradients.
 */
TT_API int tt_gate_residual_forward(void* out, const void* x, const void* gate, const void* residual,
                                    int64_t rows, int64_t cols, int64_t rows_per_batch, void* stream);
TT_API int tt_gate_residual_backward(void* dresidual, float* dgate, const void* dout, const void* gate,
                                     const void* residual, void* workspace, size_t workspace_bytes,
                                     int64_t rows, int64_t cols, int64_t rows_per_batch, void* stream);
TT_API size_t tt_gate_residual_backward_workspace_bytes(int64_t rows, int64_t cols, int64_t rows_per_batch);

/* ------------------------------------------------------------------ residual update + LayerNorm
 * The residual update of a DiT block fused with the normalisation that reads its result
 * (teletron/models/wan/wan_model.py:239-241: `x = self.gate(x, gate_msa, attn_output)`,
 * `x = x + self.cross_attn(self.norm3(x), context)`, `modulate(self.norm2(x), shift_mlp, scale_mlp)`):
 *
 *   s = x + gate * r      (gate != NULL)      or      s = x + r
 *   y = LayerNorm(s) * (1 + scale) + shift    (affine == 0: AdaLN modulation)
 *   y = LayerNorm(s) * scale + shift          (affine != 0: nn.LayerNorm weight / bias, wan_model.py:224)
 *
 * s is rounded to bf16 and it is the rounded value that is normalised, as in the unfused
 * sequence.  gate holds n_gate vectors of cols elements and scale / shift n_param vectors each,
 * where a count is 1 (shared by all batches) or rows / rows_per_batch (one per batch).
 * Vector path only: cols % 8 == 0, cols > 256, 16-byte aligned tensors (TT_ERR_UNSUPPORTED
 * otherwise; callers then run the two operations separately).  mean / rstd: optional [rows] fp32.
 *
 * Backward receives dy (gradient of y) and ds_in (gradient reaching s from its other consumers;
 * NULL = none) and the saved s:
 *   dx = ds_in + dLayerNorm(dy)      gradient of x, and of r when there is no gate
 *   dr = gate * dx, dgate = sum over rows of dx * r         (gate != NULL)
 *   dscale = sum over rows of dy * x_hat, dshift = sum over rows of dy
 * dscale, dshift, dgate: fp32 [rows / rows_per_batch, cols], one vector per batch even where the
 * parameter is shared (the caller adds the batches of a shared parameter).  Deterministic. */
TT_API int tt_residual_norm_forward(void* s, void* y, const void* x, const void* r,
                                    const void* gate, int64_t n_gate,
                                    const void* scale, const void* shift, int64_t n_param, int affine,
                                    float* mean, float* rstd,
                                    int64_t rows, int64_t cols, int64_t rows_per_batch, float eps, void* stream);
TT_API int tt_residual_norm_backward(void* dx, void* dr, float* dscale, float* dshift, float* dgate,
                                     const void* dy, const void* ds_in, const void* s, const void* r,
                                     const void* gate, int64_t n_gate, const void* scale, int64_t n_param, int affine,
                                     void* workspace, size_t workspace_bytes,
                                     int64_t rows, int64_t cols, int64_t rows_per_batch, float eps, void* stream);
TT_API size_t tt_residual_norm_backward_workspace_bytes(int64_t rows, int64_t cols, int64_t rows_per_batch, int gated);

/* ------------------------------------------------------------------ bare streaming probe
 * Measurement aid without a counterpart in the reference.  Over `bytes` bytes, with the
 * load/store policy of the kernels above, one workgroup per compute unit and no arithmetic:
 *   out, a        out[i] = a[i]                       (one read, one write)
 *   out, a, b     out[i] = a[i] ^ b[i]                (two reads, one write)
 *   a only        a is read and dropped               (out == NULL: reads on their own)
 *   out only      every 16-byte pack of out receives its own index (low 32 bits) in each of its
 *                 four words                          (a == NULL: writes on their own)
 * A benchmark runs it on the same buffers to report what each traffic mix reaches on the
 * machine at hand, next to the published HBM peak.  bytes % 16 == 0 and 16-byte aligned pointers
 * (TT_ERR_UNSUPPORTED otherwise); bytes == 0 is a no-op; out == a == NULL, or b without both
 * out and a, is TT_ERR_INVALID_ARGUMENT. */
TT_API int tt_stream_probe(void* out, const void* a, const void* b, size_t bytes, void* stream);

/* The same for one read and two writes, the traffic of tt_launch_adaln_forward (which stores
 * x_norm next to the output): out0[i] = a[i], out1[i] = ~a[i].  No counterpart in the reference.
 * All three pointers are required (TT_ERR_INVALID_ARGUMENT); sizes and alignment as above. */
TT_API int tt_stream_probe_two_outputs(void* out0, void* out1, const void* a, size_t bytes, void* stream);

/* ------------------------------------------------------------------ reference-compatible contract
 * Argument for argument the launchers the reference's pybind glue calls, plus a trailing
 * stream (the reference launches on the legacy default stream) and, for backward, the
 * workspace the reference allocates on the fly (weight_backward.cu:229).  They keep the
 * reference's saved tensors and output types:
 *   - forward also writes x_norm = bf16((x - mean) * rstd) and inv_variance = rstd [rows] fp32;
 *   - AdaLN backward reads x_norm and inv_variance (not x); scale/shift are one [cols]
 *     vector; dscale/dshift are bf16 [cols];
 *   - RMSNorm backward reads the forward *output* and reconstructs x_hat = y / weight, so a
 *     zero weight gives Inf/NaN exactly as in the reference; dweight is bf16 [cols].
 * Unlike the reference, any cols that is a multiple of 8 (up to TT_MAX_COLS) is accepted,
 * the arithmetic is fp32 with one rounding at each store, and parameter gradients are
 * reduced in fp32 before the single rounding to bf16.
 */

/* launch_adaln_forward: adaln_kernel.h:20-29, adaln_forward.cu:198-220, called from adaln_ops.cpp:16-26. */
TT_API int tt_launch_adaln_forward(void* output, void* x_norm, const void* input,
                                   const void* scale, const void* shift,
                                   int64_t rows, int64_t cols, double epsilon,
                                   float* inv_variance, void* stream);
/* launch_adaln_backward: adaln_kernel.h:36-44, adaln_backward.cu:129-151, called from adaln_ops.cpp:39-49.
 * Workspace: tt_adaln_backward_workspace_bytes(rows, cols, rows). */
TT_API int tt_launch_adaln_backward(void* dinp, void* dscale, void* dshift,
                                    const void* dout, const void* x_norm, const void* scale,
                                    const float* inv_variance, int64_t rows, int64_t cols,
                                    void* workspace, size_t workspace_bytes, void* stream);
/* launch_rms_forward: rmsnorm_kernel.h:5-12, rms_forward.cu:102-121, called from rms_ops.cpp:14-22. */
TT_API int tt_launch_rms_forward(void* output, const void* input, const void* weight,
                                 int64_t rows, int64_t cols, double epsilon,
                                 float* inv_variance, void* stream);
/* launch_rms_backward: rmsnorm_kernel.h:19-25, rms_backward.cu:91-112, called from rms_ops.cpp:34-43.
 * x_rmsnorm is the forward output.  Workspace: tt_rmsnorm_backward_workspace_bytes(rows, cols). */
TT_API int tt_launch_rms_backward(void* dinp, void* dweight,
                                  const void* dout, const void* x_rmsnorm, const void* weight,
                                  const float* inv_variance, int64_t rows, int64_t cols,
                                  void* workspace, size_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TELETRON_OP_H_ */
