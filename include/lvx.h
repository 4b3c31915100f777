/*
 * lvx.h - C ABI of the MI355X (gfx950) cross-attention hot path of LV-XAttn.
 *
 * One shared library (liblvx.so) built by hipcc; a Python, C or C++ host binds
 * these symbols directly (ctypes / dlopen).  Nothing here uses a torch type.
 *
 * Conventions
 *   - every data pointer is a DEVICE pointer owned by the caller; the library
 *     allocates nothing, keeps no pointer after a call returns and never
 *     synchronises: all work is queued on `stream` (a hipStream_t, NULL = the
 *     default stream);
 *   - 16-bit tensors are bf16 or fp16 (one type per call, "16-bit" below); strides are in ELEMENTS, the last (head_dim)
 *     stride is 1, every other stride is a multiple of 8 and every base pointer
 *     is 16-byte aligned;
 *   - q-like tensors are indexed [batch, q_head, text_row, d], kv-like tensors
 *     [batch, kv_head, visual_token, d] with Hq % Hkv == 0; q head h reads kv
 *     head h / (Hq/Hkv) (the order lv_xattn/attn.py:271-277 expands to);
 *   - LSE / delta are fp32 [B*Hq, Lq] contiguous, natural-log LSE of
 *     scale*q.k (lv_xattn/attn.py:265-268);
 *   - [row_begin, row_begin+row_count) selects the text rows one call works on:
 *     one query block of one round, or all of them at once;
 *   - return value: 0 = queued; negative = argument rejected on the host before
 *     anything was launched (LVX_ERR_*); positive = hipError_t of the launch that
 *     failed (entry points that are several launches may have queued the earlier ones;
 *     a stale error of an unrelated earlier HIP call is neither reported nor cleared).
 *     Nothing throws or aborts.  Calls are re-entrant.
 */
#ifndef LVX_H
#define LVX_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LVX_VERSION 103

#define LVX_OK 0
#define LVX_ERR_NULL (-1)        /* a required pointer is NULL */
#define LVX_ERR_ALIGN (-2)       /* pointer not 16-byte aligned / stride not a multiple of 8 */
#define LVX_ERR_SHAPE (-3)       /* non-positive or inconsistent sizes, bad row window */
#define LVX_ERR_HEAD_DIM (-4)    /* head_dim other than 16, 32, 64 or 128 */
#define LVX_ERR_DTYPE (-5)       /* dtype other than LVX_BF16 / LVX_F16 */
#define LVX_ERR_SCALE (-6)       /* scale must be finite and > 0 */
#define LVX_ERR_WORKSPACE (-7)   /* workspace missing or too small */
#define LVX_ERR_UNSUPPORTED (-8) /* valid request this build does not implement */

#define LVX_BF16 1
#define LVX_F16 2               /* the reference's dtype (lv_xattn/attn.py:226,250,268) */

/* Sizes shared by the attention entry points. */
typedef struct lvx_attn_shape {
    int32_t B, Hq, Hkv;
    int32_t D;               /* head_dim: 16, 32, 64 or 128, the values the reference names
                                (lv_xattn/attn.py:310; its Triton blocks need a power of two) */
    int32_t Lq;              /* text rows per sample (padded length)        */
    int32_t Lkv;             /* visual tokens per sample (padded length)    */
    int32_t dtype;           /* LVX_BF16 or LVX_F16: element type of q, k, v, o, dout, dq (and bf16/fp16 dk, dv) */
    float scale;             /* softmax scale, applied before the mask      */
    const int32_t* kv_len;   /* [B] valid visual tokens per sample, or NULL */
    const int32_t* kv_start; /* [B, Lq] first visible token per text row, or NULL */
    const int32_t* kv_end;   /* [B, Lq] one past the last visible token (both or neither) */
    /* Dense additive bias, fp32, added to scale * q k^T before the softmax (the tensor the
     * reference's bias_func returns, lv_xattn/attn.py:386-389, 238-241), or NULL.  Element
     * (b, h, row, key) is at bias[b*bias_stride_b + h*bias_stride_h + row*bias_stride_r + key];
     * bias_stride_h = 0 broadcasts over heads.  -inf entries mask.  No gradient is formed
     * for it (the reference forms none).  Rows are read in groups of 4 keys with 16-byte
     * loads: bias must be 16-byte aligned, the three strides multiples of 4 (LVX_ERR_ALIGN
     * otherwise), and bias_stride_r at least Lkv rounded up to a multiple of 4 (pad the rows).
     * Mask with -inf or a moderate negative (e.g. -30000), not with -FLT_MAX-sized values:
     * the backward subtracts the row's LSE from score + bias in fp32. */
    const float* bias;
    int64_t bias_stride_b, bias_stride_h, bias_stride_r;
} lvx_attn_shape;

/* A 4-d tensor with unit last stride. */
typedef struct lvx_tensor {
    void* ptr;
    int64_t stride_b, stride_h, stride_s;
} lvx_tensor;

int lvx_version(void);
const char* lvx_strerror(int code);

/*
 * Flash cross-attention forward of the selected text rows against the whole
 * local K/V shard: O (16-bit, normalised) and LSE.  Rows that see no key get
 * O = 0 and LSE = -inf.  Replaces the `_fwd_kernel` launch of one round
 * (lv_xattn/attn.py:140-268, launched at :390-400) and the per-round KV head
 * expansion (:271-277, :392-393), which happens in-kernel here.
 * kv_splits > 1 cuts the shard into that many key ranges computed by separate
 * work-groups and folded before return; it needs a workspace of
 * lvx_fwd_workspace_bytes(shape, row_count, kv_splits) bytes.
 * The bf16 kernel without a dense bias or an interval mask has two forms: a wavefront owns
 * 32 text rows, or 64 rows and its SIMD to itself (half the LDS traffic per MFMA, one
 * work-group per CU).  The second is picked when row_count is a whole number of work-group
 * row blocks and the launch has at least one work-group per CU; the environment variable
 * LVX_FWD_WIDE (0 / 1, read at every call) overrides the choice.
 * Both forms give results within the same tolerance of each other, not the same bits.
 */
int lvx_fwd(const lvx_attn_shape* shape, const lvx_tensor* q, const lvx_tensor* k,
            const lvx_tensor* v, const lvx_tensor* o, float* lse,
            int32_t row_begin, int32_t row_count, int32_t kv_splits,
            void* workspace, size_t workspace_bytes, void* stream);

/*
 * lvx_fwd whose result is merged with an incoming accumulator (o_in [like o], l_in
 * [B*Hq, Lq], only read) before it is written to (o, lse): one round's _fwd_kernel launch plus
 * its _rescale_kernel launch (lv_xattn/attn.py:390-400 and 403-419) in one call.  With key
 * splits the partials and the accumulator are folded by the same merge launch.  The kernel writes
 * (o, lse) before the merge reads (o_in, l_in): o may not overlap o_in and lse may not overlap l_in
 * over the rows of the window (LVX_ERR_SHAPE).  Workspace as for lvx_fwd.
 */
int lvx_fwd_acc(const lvx_attn_shape* shape, const lvx_tensor* q, const lvx_tensor* k, const lvx_tensor* v,
                const lvx_tensor* o_in, const float* l_in, const lvx_tensor* o, float* lse,
                int32_t row_begin, int32_t row_count, int32_t kv_splits,
                void* workspace, size_t workspace_bytes, void* stream);

size_t lvx_fwd_workspace_bytes(const lvx_attn_shape* shape, int32_t row_count, int32_t kv_splits);

/*
 * lvx_fwd for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the
 * reference.  The key-split partials go to an array inside the library
 * (LVX_NOALLOC_SCRATCH_BYTES of device memory per GPU, held until the process ends) instead
 * of a caller's workspace; the call allocates and frees nothing.  Same arguments, results
 * and return codes as lvx_fwd otherwise; LVX_ERR_WORKSPACE when
 * lvx_fwd_workspace_bytes(shape, row_count, kv_splits) exceeds the array.  The array belongs
 * to the device that is current when the call is made, which must be the stream's device.
 * All calls on one GPU share the array: calls that overlap in time on one GPU (two streams,
 * two threads) race; calls queued on one stream do not.
 */
#define LVX_NOALLOC_SCRATCH_BYTES (16u << 20)
int lvx_fwd_noalloc(const lvx_attn_shape* shape, const lvx_tensor* q, const lvx_tensor* k,
                    const lvx_tensor* v, const lvx_tensor* o, float* lse,
                    int32_t row_begin, int32_t row_count, int32_t kv_splits, void* stream);
size_t lvx_noalloc_scratch_bytes(void);

/*
 * Rescale-merge: folds a partial (o_part, l_part) over one key set into the
 * travelling accumulator (o_acc, l_acc) of the same rows, in place:
 *   L' = ln(e^La + e^Lb),  O' = Oa e^(La-L') + Ob e^(Lb-L').
 * Replaces `_rescale_kernel` (lv_xattn/attn.py:37-110, launched at :405-419),
 * evaluated with the maximum subtracted; (-inf, -inf) stays (0, -inf).
 */
int lvx_merge(const lvx_attn_shape* shape, const lvx_tensor* o_acc, float* l_acc,
              const lvx_tensor* o_part, const float* l_part,
              int32_t row_begin, int32_t row_count, void* stream);

/*
 * kv_start / kv_end [B, Lq] (int32, written): per text row the hull of the keys that
 * shape->bias leaves visible (entries other than -inf; over all heads when bias_stride_h != 0;
 * (0, 0) for a row that sees nothing).  Passed back as shape->kv_start / kv_end next to the same
 * bias, they let lvx_fwd / lvx_bwd skip the tiles outside the hull; the results do not change,
 * because a bias of -inf removes those pairs anyway.  shape->kv_start / kv_end are not read here.
 * No counterpart in the reference, which loads and adds its dense bias on every tile of a
 * block (lv_xattn/attn.py:238-241, flash_attn_kernels.py:496-512): this is the step that makes
 * a mask handed over as a bias cost what it leaves visible.
 */
int lvx_bias_hull(const lvx_attn_shape* shape, int32_t* kv_start, int32_t* kv_end, void* stream);

/*
 * Tests whether shape->bias is nothing but the interval mask lvx_bias_hull found for it:
 * *not_interval (device memory, zero on entry) is set to 1 when some entry inside a row's
 * [kv_start, kv_end) is not exactly 0 (outside the hull every entry is -inf by construction).
 * When it stays 0 the caller may drop the bias and run lvx_fwd / lvx_bwd with the intervals
 * alone - the interval-mask kernels, which read no bias at all - and get the same result.
 * No counterpart in the reference (lv_xattn/attn.py:238-241 adds whatever bias it is handed);
 * this is what lets a Llama-3.2 cross-attention mask that arrives dense, as transformers
 * builds it, run at the cost of the compact mask.
 */
int lvx_bias_is_interval(const lvx_attn_shape* shape, const int32_t* kv_start, const int32_t* kv_end,
                         int32_t* not_interval, void* stream);

/*
 * delta[b*Hq+h, row] = sum_d O * dO.  Replaces `_bwd_preprocess_do_o_dot`
 * (lv_xattn/flash_attn_kernels.py:287-329, launched at :926-942).
 */
int lvx_bwd_preprocess(const lvx_attn_shape* shape, const lvx_tensor* o, const lvx_tensor* dout,
                       float* delta, int32_t row_begin, int32_t row_count, void* stream);

/*
 * Backward of the selected text rows against the whole local shard, from the
 * saved (finally merged) LSE and delta.  Replaces `_bwd_kernel`
 * (lv_xattn/flash_attn_kernels.py:364-640, 677-819; launcher :904-1020, incl.
 * the fp32 dQ scratch and `dq.copy_` of :1020) and the host-side
 * `dk += dk_delta; dv += dv_delta` of lv_xattn/attn.py:523-524.
 *   dq     : 16-bit, rows of the window are OVERWRITTEN (windows of different
 *            rounds are disjoint, so nothing has to be accumulated);
 *   dk, dv : at Hkv heads (the group sum is taken in registers);
 *            dkv_accumulate == 0: 16-bit tensors, overwritten;
 *            dkv_accumulate == 1: fp32 tensors of the same indexing, added to;
 *   workspace : lvx_bwd_workspace_bytes(shape, row_count) bytes, 16-byte
 *            aligned; holds scale*dS (16-bit) between the kernels of the call, the row
 *            metadata and, for small windows, fp32 partial sums of dK/dV and partial tiles of dQ.
 */
int lvx_bwd(const lvx_attn_shape* shape, const lvx_tensor* q, const lvx_tensor* k,
            const lvx_tensor* v, const lvx_tensor* dout, const float* lse, const float* delta,
            const lvx_tensor* dq, const lvx_tensor* dk, const lvx_tensor* dv, int32_t dkv_accumulate,
            int32_t row_begin, int32_t row_count, void* workspace, size_t workspace_bytes, void* stream);

size_t lvx_bwd_workspace_bytes(const lvx_attn_shape* shape, int32_t row_count);

/*
 * dst(dtype, strided) = src(fp32, [B, H, L, D] contiguous): the final rounding of
 * an fp32 accumulator (the `dq.copy_(dq_accum)` of flash_attn_kernels.py:1020).
 */
int lvx_cast_f32(const float* src, const lvx_tensor* dst, int32_t B, int32_t H, int32_t L,
                 int32_t D, int32_t dtype, void* stream);

/*
 * K/V recompute from the shared visual hidden states:
 *   K[M, N] = X[M, Dm] * W_k,   V[M, N] = X[M, Dm] * W_v      (16-bit in, fp32 accumulate;
 *   `dtype`, LVX_BF16 or LVX_F16, is the element type of every matrix of the call)
 * with M = B*Lkv rows and N = Hkv*D columns, so K/V land in [B, Lkv, Hkv, D]
 * memory order.  Replaces the k_proj / v_proj nn.Linear calls inside `project`
 * (test_llama3.py:395-398) run in forward and again in backward (:197, :235).
 * w_in_major != 0: W is [Dm, N] row-major;  w_in_major == 0: W is [N, Dm]
 * row-major (torch.nn.Linear.weight).  ld* are row strides in elements.
 * w_v and v_out may both be null: a single projection, which with
 * lvx_kv_proj_norm is the text side of `project`,
 * `query_states = self.q_norm(self.q_proj(hidden_states))` (test_llama3.py:390-393).
 * The same holds for the second operand pair of lvx_dx_vis (dv, w_v) and of
 * lvx_dw_kv (dv, dw_v).
 */
int lvx_kv_proj(const void* x, int64_t ldx, const void* w_k, const void* w_v, int64_t ldw,
                int32_t w_in_major, void* k_out, void* v_out, int64_t ldkv,
                int32_t M, int32_t Dm, int32_t N, int32_t dtype, void* stream);

/*
 * The same with the k_norm of `project` (`key_states = self.k_norm(key_states)`,
 * test_llama3.py:418; MllamaTextRMSNorm of transformers 4.47.1 over head_dim)
 * applied to K in the GEMM's epilogue, per row and per head of 128 columns:
 *   x = rn(X W_k),  r = rsqrt(mean_d(x^2) + eps),  K = rn(w * rn(x * r)),  rn = round to dtype.
 * N must be a multiple of 128.  k_norm_w: 128 weights of that type, 16-byte aligned.
 * Optional outputs for the norm's backward (null: not written):
 *   k_raw  : x, indexed like k_out (row stride ldkv);
 *   k_rstd : r, fp32 [M, N / 128].
 */
int lvx_kv_proj_norm(const void* x, int64_t ldx, const void* w_k, const void* w_v, int64_t ldw,
                     int32_t w_in_major, void* k_out, void* v_out, int64_t ldkv,
                     int32_t M, int32_t Dm, int32_t N, const void* k_norm_w, float eps,
                     void* k_raw, float* k_rstd, int32_t dtype, void* stream);

/*
 * Backward of that norm (what autograd derives for test_llama3.py:418 when the
 * K/V gradients are propagated, which the reference's wrapper does not do,
 * :243): with xh = k_raw * r and g = dk * w, per row and head
 *   dk_raw = r * (g - xh * mean_d(g * xh)),   dw[d] += sum over rows, heads of dk * rn(xh).
 * dk_raw may alias dk.  dw: fp32 [128], ADDED to (null: not wanted).
 */
int lvx_k_norm_bwd(const void* dk, int64_t lddk, const void* k_raw, int64_t ldk, const float* k_rstd,
                   const void* k_norm_w, void* dk_raw, int64_t lddk_raw, float* dw,
                   int32_t M, int32_t N, int32_t dtype, void* stream);

/*
 * dX[M, Dm] = dK[M, N] * W_k^T + dV[M, N] * W_v^T  (no counterpart in the
 * reference, whose wrapper drops this gradient: test_llama3.py:243).
 */
int lvx_dx_vis(const void* dk, const void* dv, int64_t lddkv, const void* w_k, const void* w_v,
               int64_t ldw, int32_t w_in_major, void* dx, int64_t lddx,
               int32_t M, int32_t Dm, int32_t N, int32_t dtype, void* stream);

/*
 * dW_k = X^T dK, dW_v = X^T dV in the layout of W (see w_in_major); the weight
 * gradients the recompute path needs to train the projections.
 */
int lvx_dw_kv(const void* x, int64_t ldx, const void* dk, const void* dv, int64_t lddkv,
              void* dw_k, void* dw_v, int64_t ldw, int32_t w_in_major,
              int32_t M, int32_t Dm, int32_t N, int32_t dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* LVX_H */
