/*
 * xpu_graph_amd.h -- C ABI of the MI355X (gfx950) kernel library behind the
 * `mi355x` target of the xpu_graph FX/Aten compiler.
 *
 * Every entry point
 *   - takes plain device pointers, sizes, strides (in ELEMENTS unless the name
 *     says bytes) and a HIP stream (`void*` == hipStream_t, NULL = default);
 *   - only enqueues work on that stream: it never allocates, never frees and
 *     never synchronises, so it can be recorded into a HIP graph;
 *   - validates its arguments on the host and returns XG_OK (0) or a negative
 *     xg_status code without launching anything when they do not fit what the
 *     kernel assumes;  xg_status_string() names the code.
 *
 * The reference (XPU-Forces/xpu_graph, 100 % Python) has no FFI of its own: its
 * target packages call vendor operator libraries.  Each declaration below cites
 * the reference call site whose arithmetic it replaces.
 */
#ifndef XPU_GRAPH_AMD_H
#define XPU_GRAPH_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* xg_stream_t; /* hipStream_t */

typedef enum {
  XG_OK = 0,
  XG_ERR_BAD_DTYPE = -1,   /* dtype / dtype combination has no kernel            */
  XG_ERR_BAD_SHAPE = -2,   /* negative or inconsistent sizes / strides           */
  XG_ERR_BAD_ALIGN = -3,   /* pointer or stride alignment the kernel cannot take */
  XG_ERR_NULL_PTR = -4,    /* a required pointer is NULL                         */
  XG_ERR_TOO_LARGE = -5,   /* size beyond what the entry point supports          */
  XG_ERR_LAUNCH = -6,      /* hipLaunchKernel reported an error                  */
  XG_ERR_BAD_ARG = -7      /* other invalid argument (enum value, flag)          */
} xg_status;

typedef enum { XG_F32 = 0, XG_F16 = 1, XG_BF16 = 2, XG_FP8_E4M3 = 3 } xg_dtype;

typedef enum { XG_ACT_NONE = 0, XG_ACT_RELU = 1, XG_ACT_GELU = 2, XG_ACT_SILU = 3, XG_ACT_SIGMOID = 4 } xg_act;

/* Library version (major*10000 + minor*100 + patch) and status text. */
int xg_version(void);
const char* xg_status_string(int status);

/* ---------------------------------------------------------------------------
 * Row normalisation.  x, y, h, res are [rows, cols] with unit column stride;
 * x_stride / res_stride are row strides in elements, outputs are contiguous.
 * w and b are [cols] of dtype `wb_dtype`, which must equal `dtype` or XG_F32.
 * Statistics and the affine transform are computed in fp32 and rounded once
 * to `dtype`.
 *
 * xg_rms_norm:   y = x * rsqrt(mean(x^2) + eps) * w            (w may be NULL)
 *   replaces DefaultRMSNorm.forward
 *   (src/xpu_graph/passes/patterns/utils/default_replacements.py:19-25) and the
 *   vendor calls torch_mlu_ops.fused_rms_norm
 *   (passes/patterns/targets/mlu/structure_replacements/norm_modules.py:4-10),
 *   torch_npu.npu_rms_norm
 *   (passes/patterns/targets/npu/structure_replacements/rms_norm_module.py:6-10).
 *
 * xg_layer_norm: y = (x - mean) * rsqrt(var + eps) * w + b     (w, b may be NULL)
 *   replaces DefaultLayerNorm.forward (default_replacements.py:28-36) and
 *   torch_mlu_ops.fused_layer_norm (norm_modules.py:13-21).
 *
 * xg_add_rms_norm / xg_add_layer_norm: h = round_to_dtype(x + res), then the
 *   norm of h (statistics taken of the ROUNDED h, as the unfused graph does).
 *   h_out may be NULL (store_output_before_norm == False).
 *   replace FusedNormReplacement.forward
 *   (passes/patterns/targets/mlu/fuse_add_norm.py:21-83) and the op
 *   torch_npu_triton::fused_add_rmsnorm
 *   (passes/patterns/targets/npu/triton_kernel/fused_add_rmsnorm.py:8-72).
 * ------------------------------------------------------------------------- */
int xg_rms_norm(const void* x, const void* w, void* y, int64_t rows, int64_t cols, int64_t x_stride, float eps,
                int dtype, int wb_dtype, xg_stream_t stream);
int xg_layer_norm(const void* x, const void* w, const void* b, void* y, int64_t rows, int64_t cols,
                  int64_t x_stride, float eps, int dtype, int wb_dtype, xg_stream_t stream);
int xg_add_rms_norm(const void* x, const void* res, const void* w, void* y, void* h_out, int64_t rows,
                    int64_t cols, int64_t x_stride, int64_t res_stride, float eps, int dtype, int wb_dtype,
                    xg_stream_t stream);
int xg_add_layer_norm(const void* x, const void* res, const void* w, const void* b, void* y, void* h_out,
                      int64_t rows, int64_t cols, int64_t x_stride, int64_t res_stride, float eps, int dtype,
                      int wb_dtype, xg_stream_t stream);

/* ---------------------------------------------------------------------------
 * Backward of xg_rms_norm / xg_add_rms_norm for training graphs (the reference
 * differentiates its fused norms through AOT autograd:
 * tests/common/test_fuse_rmsnorm.py:125-157, tests/common/test_training.py).
 *   h = x (+ res, rounded to `dtype` as the forward rounds it), r = rsqrt(mean(h^2) + eps), hhat = h r
 *   gx[rows, cols] (contiguous) = r (gy w - hhat mean(gy w hhat)) (+ gh)   -- the gradient of x, and of res
 *   gw_part[n_blocks, cols] fp32: block b's share of sum_rows(gy hhat); the caller adds the n_blocks rows
 *     (NULL when the weight gradient is not wanted; needs w).
 * res, w, gh may be NULL.  n_blocks workgroups split the rows (1 <= n_blocks <= 65535; when rows < n_blocks the
 * rows beyond `rows` of gw_part are left unwritten, so pass n_blocks <= rows).  cols a multiple of 8 (4 for fp32)
 * and at most 16384 (8192 for fp32); strides in elements, multiples of the same.
 * ------------------------------------------------------------------------- */
int xg_rms_norm_bwd(const void* x, const void* res, const void* w, const void* gy, const void* gh, void* gx, float* gw_part,
                    int64_t rows, int64_t cols, int64_t x_stride, int64_t res_stride, int64_t gy_stride, int64_t gh_stride,
                    float eps, int dtype, int w_dtype, int n_blocks, xg_stream_t stream);

/* ---------------------------------------------------------------------------
 * Backward of xg_layer_norm / xg_add_layer_norm, same conventions (the
 * reference's LayerNorm training cases: tests/common/test_fuse_layernorm.py).
 *   h = x (+ res), mu = mean(h), r = rsqrt(mean((h - mu)^2) + eps), hhat = (h - mu) r
 *   gx = r (gy w - mean(gy w) - hhat mean(gy w hhat)) (+ gh)
 *   gw_part[n_blocks, cols] fp32: shares of sum_rows(gy hhat) (needs w);
 *   gb_part[n_blocks, cols] fp32: shares of sum_rows(gy), the bias gradient; either may be NULL.
 * ------------------------------------------------------------------------- */
int xg_layer_norm_bwd(const void* x, const void* res, const void* w, const void* gy, const void* gh, void* gx, float* gw_part,
                      float* gb_part, int64_t rows, int64_t cols, int64_t x_stride, int64_t res_stride, int64_t gy_stride,
                      int64_t gh_stride, float eps, int dtype, int w_dtype, int n_blocks, xg_stream_t stream);

/* ---------------------------------------------------------------------------
 * Column slice + concatenate (bit-exact byte mover, dtype-agnostic).
 *
 * For every row r < rows and every chunk i < n_chunks, copies `chunk_bytes`
 * bytes from   src + r*src_row_bytes + table[i].src_off
 *        to    outs[table[i].out_id] + r*out_row_bytes[out_id] + table[i].dst_off.
 * `table` lives in DEVICE memory (built once by the caller for a static slice
 * list); chunk_bytes is one of 1,2,4,8,16.  src, src_row_bytes, every src_off,
 * every out pointer / out_row_bytes / dst_off must be multiples of
 * min(chunk_bytes, 4) for the source side and of chunk_bytes for the output
 * side.  n_outs <= XG_SLICE_CAT_MAX_OUTS.
 *
 * The table is device memory, so xg_slice_cat cannot look at it without a
 * synchronisation: an entry outside a row is an out-of-bounds access, not an
 * error code.  xg_slice_cat_check_table() validates a HOST copy of the table
 * once, when it is built: every chunk must lie inside the first
 * `src_row_valid_bytes` bytes of a source row and inside the first
 * `out_row_valid_bytes[out_id]` bytes of a row of its output, with the
 * alignment stated above; it launches nothing.  The reference builds its index
 * tensor from the matched slice list at module construction
 * (FuseSliceCatSameInputModule_v2.__init__, structure_replacements/__init__.py:66-95)
 * and has no such check.
 *
 * replaces torch_mlu_triton::fused_slice_cat
 *   (passes/patterns/targets/mlu/triton_kernel/fused_slice_cat.py:10-73; one
 *   output) and torch_mlu_triton::fused_slice_low_v2
 *   (.../triton_kernel/fused_slice_v2.py:9-114; several outputs in one launch).
 * ------------------------------------------------------------------------- */
#define XG_SLICE_CAT_MAX_OUTS 32
typedef struct {
  int32_t src_off; /* byte offset inside a source row */
  int32_t dst_off; /* byte offset inside a row of the chosen output */
  int32_t out_id;  /* which output */
  int32_t pad;
} xg_chunk;
int xg_slice_cat(const void* src, int64_t src_row_bytes, int64_t rows, void* const* outs,
                 const int64_t* out_row_bytes, int n_outs, const xg_chunk* table_dev, int64_t n_chunks,
                 int chunk_bytes, xg_stream_t stream);
int xg_slice_cat_check_table(const xg_chunk* table_host, int64_t n_chunks, int chunk_bytes, int64_t src_row_valid_bytes,
                             const int64_t* out_row_valid_bytes, int n_outs);

/* ---------------------------------------------------------------------------
 * add-N: out = ((t0 + t1) + t2) + ... strictly left to right, fp32 accumulate,
 * one rounding to `dtype` at the end.  `inputs` is a HOST array of n device
 * pointers to contiguous tensors of `numel` elements.  n >= 1.
 * replaces the stack + sum(dim 0) that FusedAddN emits
 *   (passes/patterns/common/fuse_addn.py:27-76).
 * ------------------------------------------------------------------------- */
int xg_addn(const void* const* inputs, int n, void* out, int64_t numel, int dtype, xg_stream_t stream);

/* ---------------------------------------------------------------------------
 * combo-sum: n_jobs independent reductions in one launch.  Job j reduces a
 * contiguous [s0, s1, s2] tensor over dim 1 (-> [s0, s2]) or dim 2 (-> [s0, s1]),
 * fp32 accumulate in index order, one rounding.  All arrays are HOST arrays of
 * length n_jobs; n_jobs <= XG_COMBO_SUM_MAX_JOBS.
 * replaces torch_mlu_triton::fused_sum_3d_input
 *   (passes/patterns/targets/mlu/triton_kernel/fused_sum_3d.py:84-205).
 * ------------------------------------------------------------------------- */
#define XG_COMBO_SUM_MAX_JOBS 64
int xg_combo_sum(const void* const* inputs, void* const* outputs, const int64_t* s0, const int64_t* s1,
                 const int64_t* s2, int n_jobs, int dim, int dtype, xg_stream_t stream);

/* ---------------------------------------------------------------------------
 * slice -> sum -> cat: out[b, i * cols + c] = sum over r in [starts[i], ends[i]) of
 * x[b, r, c]; x is [batch, rows, cols] with unit column stride and the given batch
 * and row strides (elements), out is a contiguous [batch, n_slices * cols]; fp32
 * accumulate in row order, one rounding.  `starts` / `ends` are HOST arrays of
 * n_slices <= XG_SLICE_SUM_MAX_SLICES row bounds inside [0, rows].
 * replaces torch_mlu_triton::fuse_slice_sum_cat as called by SliceSumCatOperation
 *   (passes/patterns/targets/mlu/fuse_sum_cat.py:73-115).
 * ------------------------------------------------------------------------- */
#define XG_SLICE_SUM_MAX_SLICES 64
int xg_slice_sum_cat(const void* x, void* out, int64_t batch, int64_t rows, int64_t cols, int64_t x_batch_stride,
                     int64_t x_row_stride, const int32_t* starts, const int32_t* ends, int n_slices, int dtype,
                     xg_stream_t stream);

/* ---------------------------------------------------------------------------
 * SwiGLU gate: y[r, c] = silu(x[r, c]) * x[r, d + c], x is [rows, 2d] with row
 * stride x_stride, y is contiguous [rows, d]; fp32 math.
 * replaces torch_npu_triton::fused_silu_mul
 *   (passes/patterns/targets/npu/triton_kernel/fused_silu_mul.py:8-60).
 * xg_silu_mul2 takes gate and up as two separate [rows, d] tensors.
 * xg_silu_mul2_bwd: the gradients of xg_silu_mul2 for training graphs (the
 *   reference differentiates its fused gate through AOT autograd,
 *   tests/common/test_training.py): d_gate = gy * up * s (1 + gate (1 - s)),
 *   s = sigmoid(gate); d_up = gy * silu(gate); five contiguous tensors of n
 *   elements, fp32 math, one rounding per output.
 * ------------------------------------------------------------------------- */
int xg_silu_mul(const void* x, void* y, int64_t rows, int64_t d, int64_t x_stride, int dtype,
                xg_stream_t stream);
int xg_silu_mul2(const void* gate, const void* up, void* y, int64_t rows, int64_t d, int64_t gate_stride,
                 int64_t up_stride, int dtype, xg_stream_t stream);
int xg_silu_mul2_bwd(const void* gate, const void* up, const void* gy, void* d_gate, void* d_up, int64_t n, int dtype,
                     xg_stream_t stream);

/* ---------------------------------------------------------------------------
 * An activation on its own and its backward, for the dense layer of a training
 * graph (the reference's FusedDenseLayer takes relu / gelu / silu / sigmoid,
 * passes/patterns/structure/fuse_denselayer.py; in a differentiated graph the
 * layer keeps its pre-activation z as eager does, so the backward is one pass
 * over z and gy instead of a second product):
 *   xg_activation:     y[i]  = act(x[i])
 *   xg_activation_bwd: gz[i] = gy[i] * act'(z[i])
 * n contiguous elements, fp32 math, one rounding; `act` one of XG_ACT_RELU,
 * _GELU (erf form), _SILU, _SIGMOID (XG_ACT_NONE: XG_ERR_BAD_ARG).
 * ------------------------------------------------------------------------- */
int xg_activation(const void* x, void* y, int64_t n, int act, int dtype, xg_stream_t stream);
int xg_activation_bwd(const void* z, const void* gy, void* gz, int64_t n, int act, int dtype, xg_stream_t stream);

/* ---------------------------------------------------------------------------
 * Gated dense layer (SwiGLU): out[M, N] = silu(a w_gate^T) * (a w_up^T), both
 * weights [N, K] with unit K stride and row stride ldb, a [M, K] with row stride
 * lda, out contiguous [M, N]; bf16 or f16, fp32 accumulation; each projection is
 * rounded to `dtype` before the gate is applied, so the result is bit-identical
 * to two xg_dense calls followed by xg_silu_mul2.  K must be a multiple of 64.
 * No counterpart in the reference: it fuses what its test writes as two linear
 * layers and a silu * mul (tests/npu/test_silu_mul.py:8-16 after two
 * CustomDenseLayer calls, structure/custom_denselayer.py:46-128).
 * ------------------------------------------------------------------------- */
int xg_dense_glu(const void* a, const void* w_gate, const void* w_up, void* out, int64_t M, int64_t N, int64_t K,
                 int64_t lda, int64_t ldb, int dtype, xg_stream_t stream);
/* xg_dense_glu that also writes the two rounded projections (gate_out = a Wg^T, up_out = a Wu^T, [M,N] each, the
 * values the gate was computed from), for training graphs: the backward needs them and would otherwise run both
 * projections again.  Same kernel, two more stores per output element. */
int xg_dense_glu_save(const void* a, const void* w_gate, const void* w_up, void* out, void* gate_out, void* up_out,
                      int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int dtype, xg_stream_t stream);

/* ---------------------------------------------------------------------------
 * Dense layer: out[M,N] = act(a[M,K] @ B + bias (+ residual)), fp32 accumulate.
 *   a: row-major, row stride lda.  B is [K,N] row-major with row stride ldb when
 *   b_trans == 0, or the transpose of a row-major [N,K] (row stride ldb) when
 *   b_trans == 1 (the nn.Linear weight layout).
 *   bias: NULL or [N] (dtype `dtype` or XG_F32 via bias_dtype).
 *   residual: NULL or [M,N] row stride ldr, added before the activation.
 *   dtype: XG_BF16, XG_F16 or XG_F32 (inputs and output).  16-bit types use
 *   the 32x32x16 MFMA, fp32 the 32x32x2 fp32 MFMA (plain IEEE fp32 products and
 *   sums: no reduced-precision passes); fp32 is the dtype of the reference's
 *   dense-layer tests (tests/mlu/test_custom_denselayer.py:11).  K, lda, ldb,
 *   ldr multiples of 8 elements (4 for fp32), N a multiple of 8.
 *   xg_dense_batched and xg_dense_at take the 16-bit types only.
 * replaces torch_mlu_ops.matmul as called by DenseLayerModule.forward
 *   (passes/patterns/targets/mlu/structure_replacements/dense_layer_modules.py:4-56).
 *
 * xg_dense_batched: `batch` independent layers in ONE launch (batch entry on
 *   the second grid axis, same tiles and kernels as xg_dense).  Entry z reads
 *   a + z*stride_a, b + z*stride_b, bias + z*stride_bias (0: one bias for all),
 *   residual + z*stride_res and writes out + z*stride_out, all strides in
 *   elements and multiples of 8; each entry's out is [M,N] contiguous.
 *   batch <= 65535.
 * replaces torch_mlu_ops.batch_matmul as called by BatchDenseLayerModule.forward
 *   (passes/patterns/targets/mlu/structure_replacements/dense_layer_modules.py:71-111).
 *
 * xg_dense_at: out[M,N] = a_t^T @ b (+ residual) with a_t [K,M] (row stride
 *   lda) and b [K,N] (row stride ldb): the left operand arrives transposed, as
 *   the weight gradient of a dense layer does (dW^T = dY^T X: a_t = dY [tokens,
 *   out_features], b = X [tokens, in_features]).  M, N, lda, ldb, ldr multiples
 *   of 8; any K.  fp32 accumulation, one rounding.
 * replaces the mm(t(grad), x) of the backward graph the reference leaves to
 *   the device's own matmul (tests/common/test_training.py:1-80 is its bar).
 *
 * xg_dense_fp8: a_q [M,K] and b_q ([K,N] or [N,K], as above) are OCP e4m3fn
 *   bytes; out = act((a_q @ b_q) * a_scale * b_scale[n] + bias) in `out_dtype`
 *   (XG_BF16 / XG_F16 / XG_F32).  b_scale is f32[N], bias f32-or-out_dtype.
 *   No counterpart in the reference (it has no fp8 path).
 * ------------------------------------------------------------------------- */
int xg_dense(const void* a, const void* b, const void* bias, const void* residual, void* out, int64_t M,
             int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldr, int b_trans, int act, int dtype,
             int bias_dtype, xg_stream_t stream);
int xg_dense_batched(const void* a, const void* b, const void* bias, const void* residual, void* out, int64_t batch,
                     int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldr, int64_t stride_a,
                     int64_t stride_b, int64_t stride_bias, int64_t stride_res, int64_t stride_out, int b_trans,
                     int act, int dtype, int bias_dtype, xg_stream_t stream);
int xg_dense_at(const void* a_t, const void* b, const void* residual, void* out, int64_t M, int64_t N, int64_t K,
                int64_t lda, int64_t ldb, int64_t ldr, int dtype, xg_stream_t stream);
int xg_dense_fp8(const void* a_q, const void* b_q, const float* a_scale_dev, const float* b_scale_dev,
                 const void* bias, void* out, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
                 int b_trans, int act, int out_dtype, int bias_dtype, xg_stream_t stream);

/* ---------------------------------------------------------------------------
 * Scaled dot-product attention, optional causal mask, no dropout.
 *   q [B,H,Sq,D], k/v [B,Hkv,Skv,D], out [B,H,Sq,D]; strides in elements for
 *   batch, head and sequence; the D axis has unit stride; D in {64, 128}.
 *   softmax in fp32 with running max; causal hides key j from query i when
 *   j > i (the is_causal=True convention of torch, top-left aligned).
 * replaces aten.scaled_dot_product_attention as emitted by FusedSDPA
 *   (passes/patterns/common/fuse_scaled_dot_product_attention.py:184-234).
 * ------------------------------------------------------------------------- */
int xg_sdpa(const void* q, const void* k, const void* v, void* out, int64_t B, int64_t H, int64_t Hkv,
            int64_t Sq, int64_t Skv, int64_t D, const int64_t q_strides[3], const int64_t k_strides[3],
            const int64_t v_strides[3], const int64_t o_strides[3], float scale, int causal, int dtype,
            xg_stream_t stream);

/* ---------------------------------------------------------------------------
 * xg_sdpa with the two operands the general attn_mask form of FusedSDPA carries
 * (fuse_scaled_dot_product_attention.py:184-234, `attn_mask=` and a tensor
 * `scale`):
 *   mask: NULL or an additive mask, element [b,h,i,j] at
 *     mask + mask_strides[0]*b + mask_strides[1]*h + mask_strides[2]*i + j
 *     (strides in elements, 0 = broadcast along that axis), dtype `mask_dtype`
 *     = `dtype` or XG_F32; it is added to q.k^T * scale before the softmax.
 *     A row whose every key is masked with -inf comes out as NaN, as in eager.
 *   scale_dev: NULL, or a one-element fp32 DEVICE tensor that holds the scale;
 *     the kernel reads it (no host read, no synchronisation) and `scale` is
 *     ignored.  Replaces SDPAWrappedScale.forward, which reads the tensor with
 *     .item() (passes/patterns/utils/default_replacements.py:39-55).
 * `causal` may be combined with a mask.
 * ------------------------------------------------------------------------- */
int xg_sdpa_masked(const void* q, const void* k, const void* v, void* out, const void* mask,
                   const int64_t mask_strides[3], int mask_dtype, const float* scale_dev, int64_t B, int64_t H,
                   int64_t Hkv, int64_t Sq, int64_t Skv, int64_t D, const int64_t q_strides[3],
                   const int64_t k_strides[3], const int64_t v_strides[3], const int64_t o_strides[3], float scale,
                   int causal, int dtype, xg_stream_t stream);

/* ---------------------------------------------------------------------------
 * Attention for graphs that are differentiated (the reference compiles
 * training graphs through AOT autograd and leaves attention's backward to the
 * device's own kernels: compiler.py:105-180, tests/common/test_training.py).
 *   xg_sdpa_lse: xg_sdpa that also writes lse [B,H,Sq] fp32, the natural-log
 *     sum of exponentials of every query row's scaled (and causally masked)
 *     scores; -inf for a row that sees no key.
 *   xg_sdpa_backward: dq [B,H,Sq,D], dk and dv [B,Hkv,Skv,D] (in `dtype`,
 *     each with its own batch / head / sequence strides like the inputs, so a
 *     gradient can be written in the layout of the tensor it belongs to; rows
 *     of D contiguous elements that do not overlap) from q, k, v, the
 *     forward's out and lse, and d_out (strides as in xg_sdpa; d_out has its
 *     own).  The probabilities are recomputed tile by
 *     tile from lse: no [Sq,Skv] temporary.  With Hkv < H the gradients of a
 *     key/value head are summed over its query heads inside the kernel.  Two
 *     launches on `stream`; results do not depend on scheduling (no atomics).
 *     delta_ws: [B,H,Sq] fp32 workspace supplied by the caller (row sums of
 *     d_out * out, written by the first launch and read by the second).
 * ------------------------------------------------------------------------- */
int xg_sdpa_lse(const void* q, const void* k, const void* v, void* out, float* lse, int64_t B, int64_t H, int64_t Hkv,
                int64_t Sq, int64_t Skv, int64_t D, const int64_t q_strides[3], const int64_t k_strides[3],
                const int64_t v_strides[3], const int64_t o_strides[3], float scale, int causal, int dtype,
                xg_stream_t stream);
int xg_sdpa_backward(const void* q, const void* k, const void* v, const void* out, const void* d_out, const float* lse,
                     void* dq, void* dk, void* dv, float* delta_ws, int64_t B, int64_t H, int64_t Hkv, int64_t Sq,
                     int64_t Skv, int64_t D, const int64_t q_strides[3], const int64_t k_strides[3],
                     const int64_t v_strides[3], const int64_t o_strides[3], const int64_t do_strides[3],
                     const int64_t dq_strides[3], const int64_t dk_strides[3], const int64_t dv_strides[3], float scale,
                     int causal, int dtype, xg_stream_t stream);

/* ---------------------------------------------------------------------------
 * The two calls above for the attn_mask / tensor-scale form (xg_sdpa_masked):
 *   xg_sdpa_masked_lse: xg_sdpa_masked that also writes lse [B,H,Sq] fp32.
 *   xg_sdpa_backward_masked: xg_sdpa_backward with the forward's `mask`
 *     (NULL or an additive mask, indexed as in xg_sdpa_masked) and `scale_dev`
 *     (NULL or the one-element device scale).  dq, dk, dv only: the mask and
 *     the scale tensor get no gradient.  A row that the mask hides completely
 *     gives NaN gradients, as its forward result is NaN.
 * replaces the Aten backward of the attn_mask form FusedSDPA emits
 *   (passes/patterns/common/fuse_scaled_dot_product_attention.py:184-234) in
 *   training graphs.
 * ------------------------------------------------------------------------- */
int xg_sdpa_masked_lse(const void* q, const void* k, const void* v, void* out, float* lse, const void* mask,
                       const int64_t mask_strides[3], int mask_dtype, const float* scale_dev, int64_t B, int64_t H,
                       int64_t Hkv, int64_t Sq, int64_t Skv, int64_t D, const int64_t q_strides[3],
                       const int64_t k_strides[3], const int64_t v_strides[3], const int64_t o_strides[3], float scale,
                       int causal, int dtype, xg_stream_t stream);
int xg_sdpa_backward_masked(const void* q, const void* k, const void* v, const void* out, const void* d_out,
                            const float* lse, const void* mask, const int64_t mask_strides[3], int mask_dtype,
                            const float* scale_dev, void* dq, void* dk, void* dv, float* delta_ws, int64_t B, int64_t H,
                            int64_t Hkv, int64_t Sq, int64_t Skv, int64_t D, const int64_t q_strides[3],
                            const int64_t k_strides[3], const int64_t v_strides[3], const int64_t o_strides[3],
                            const int64_t do_strides[3], const int64_t dq_strides[3], const int64_t dk_strides[3],
                            const int64_t dv_strides[3], float scale, int causal, int dtype, xg_stream_t stream);

/* ---------------------------------------------------------------------------
 * xg_sdpa / xg_sdpa_masked (no causal flag) for a decode step: Sq <= 32 query
 * rows per head against long K / V.  The keys are split over workgroups (and the query
 * heads of one key/value head share a workgroup when H / Hkv * Sq <= 32), so
 * K and V stream at memory speed instead of through B * H compute units.
 *   lse: NULL or [B,H,Sq] fp32 as in xg_sdpa_lse.
 *   mask, mask_strides, mask_dtype, scale_dev: as in xg_sdpa_masked (NULL: none).
 *   workspace: NULL or `workspace_floats` fp32 of device memory for the partial
 *     results of the key ranges; xg_sdpa_decode_workspace_floats gives the size
 *     that allows the preferred split (0: none needed).  With less, the keys
 *     are split into as many ranges as fit, down to one.
 *   Sq > 32: XG_ERR_BAD_SHAPE (use xg_sdpa).
 * replaces aten.scaled_dot_product_attention as emitted by FusedSDPA
 *   (passes/patterns/common/fuse_scaled_dot_product_attention.py:184-234) for
 *   the shapes of incremental decoding.
 * ------------------------------------------------------------------------- */
int64_t xg_sdpa_decode_workspace_floats(int64_t B, int64_t H, int64_t Hkv, int64_t Sq, int64_t Skv, int64_t D);
int xg_sdpa_decode(const void* q, const void* k, const void* v, void* out, float* lse, const void* mask,
                   const int64_t mask_strides[3], int mask_dtype, const float* scale_dev, float* workspace,
                   int64_t workspace_floats, int64_t B, int64_t H, int64_t Hkv, int64_t Sq, int64_t Skv, int64_t D,
                   const int64_t q_strides[3], const int64_t k_strides[3], const int64_t v_strides[3],
                   const int64_t o_strides[3], float scale, int dtype, xg_stream_t stream);

/* ---------------------------------------------------------------------------
 * xg_sdpa_backward without the workspace argument, for callers that cannot
 * allocate device memory (code under HIP graph capture, serving loops and
 * harnesses that forbid hipMalloc).  No counterpart in the reference.  The
 * delta workspace is an 8 MiB array that lives in the library's device image,
 * one per GPU, from load until the process ends: B * H * Sq must not exceed
 * 2 097 152 query rows (XG_ERR_TOO_LARGE beyond that: use xg_sdpa_backward).
 * The call allocates and frees nothing.  The first call on a GPU also looks
 * up the array's device address and raises the kernels' LDS limit (host-side
 * set-up, no stream work): make it outside a stream capture; every later call
 * on that GPU only enqueues the two kernels.  Every call on a GPU uses that GPU's
 * one array: calls that overlap in time on the same GPU (different streams)
 * race; calls on one stream are ordered and need nothing cleared in between
 * (each call writes every row of the workspace that it later reads).
 * Results are bit-identical to xg_sdpa_backward.
 * ------------------------------------------------------------------------- */
int xg_sdpa_backward_static(const void* q, const void* k, const void* v, const void* out, const void* d_out,
                            const float* lse, void* dq, void* dk, void* dv, int64_t B, int64_t H, int64_t Hkv,
                            int64_t Sq, int64_t Skv, int64_t D, const int64_t q_strides[3],
                            const int64_t k_strides[3], const int64_t v_strides[3], const int64_t o_strides[3],
                            const int64_t do_strides[3], const int64_t dq_strides[3], const int64_t dk_strides[3],
                            const int64_t dv_strides[3], float scale, int causal, int dtype, xg_stream_t stream);

/* ---------------------------------------------------------------------------
 * Rotary position embedding, rotate-half convention:
 *   out = x * cos + cat(-x[..., D/2:], x[..., :D/2]) * sin      (fp32 math, one rounding)
 *   x, out [B,H,S,D] with element strides for batch, head, sequence (D has unit stride, D % 16 == 0);
 *   cos, sin [S,D] tables with row stride `table_stride`, dtype `table_dtype` = `dtype` or XG_F32.
 * No counterpart in the reference (it has no rotary-embedding pattern): replaces the eager
 *   mul / slice / neg / cat / mul / add subgraph of the Llama block of benchmark config 5.
 * ------------------------------------------------------------------------- */
int xg_rope(const void* x, const void* cos_table, const void* sin_table, void* out, int64_t B, int64_t H, int64_t S,
            int64_t D, const int64_t x_strides[3], const int64_t o_strides[3], int64_t table_stride, int dtype,
            int table_dtype, xg_stream_t stream);

/* ---------------------------------------------------------------------------
 * Plain device copy of `bytes` bytes (16-byte aligned), used as the known-size
 * yardstick that scales the FETCH_SIZE / WRITE_SIZE profiler counters.
 * ------------------------------------------------------------------------- */
int xg_copy_bytes(const void* src, void* dst, int64_t bytes, xg_stream_t stream);

/* ---------------------------------------------------------------------------
 * Shader-clock probe for benchmarks: one wavefront that, for each of
 * `n_windows` windows of `window_ticks` ticks of the constant-rate wall clock
 * (xg_wall_clock_khz, 100 MHz on gfx950), writes out[2w] = shader-clock ticks
 * and out[2w + 1] = wall-clock ticks that went by.  Launched on a second
 * stream beside the kernel under test, it tells the engine clock the GPU
 * sustains under that kernel: out[2w] / out[2w + 1] x wall-clock rate.
 *   out: device memory, 2 x n_windows uint64; n_windows <= 65536;
 *   0 < window_ticks <= 1000000.  Every window ends after a bounded number
 *   of polls, so the kernel always finishes.
 * No counterpart in the reference.
 * ------------------------------------------------------------------------- */
int xg_clock_probe(uint64_t* out, int n_windows, int64_t window_ticks, xg_stream_t stream);
int64_t xg_wall_clock_khz(void);

#ifdef __cplusplus
}
#endif
#endif /* XPU_GRAPH_AMD_H */
