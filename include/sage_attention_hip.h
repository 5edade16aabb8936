/*
 * C ABI of libsage_attention_hip.so: FlagAttention's SageAttention path on MI355X (gfx950), and the
 * dense 16-bit attention forward that shares its kernel.
 *
 * Plain pointers, sizes and strides only; no framework types.  All pointers are device
 * pointers on the current HIP device unless stated otherwise; strides are in ELEMENTS and the
 * innermost (head_dim) stride must be 1.  Tensors are described in the logical order
 * (batch, head, sequence, head_dim); the reference's "HND" / "NHD" layouts differ only in
 * which physical stride is passed as stride_h / stride_n.
 *
 * Every entry point enqueues work on `stream` (a hipStream_t passed as void*) and returns
 * without synchronising.  Nothing is allocated or freed; outputs and the K-mean workspace are
 * owned by the caller.  Return value: 0 on success, a negative SAGE_E_* code on a rejected call
 * (nothing was launched); sage_hip_last_error() then returns a message for the calling thread.
 */
#ifndef SAGE_ATTENTION_HIP_H
#define SAGE_ATTENTION_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum sage_dtype { SAGE_F16 = 0, SAGE_BF16 = 1, SAGE_F32 = 2 };
enum sage_mask_kind { SAGE_MASK_NONE = 0, SAGE_MASK_BOOL = 1, SAGE_MASK_F32 = 2, SAGE_MASK_F16 = 3, SAGE_MASK_BF16 = 4,
                      SAGE_MASK_BOOL_PADDED = 5, SAGE_MASK_BOOL_PADDED_CAUSAL = 6, SAGE_MASK_F16_PADDED = 7,
                      SAGE_MASK_BF16_PADDED = 8, SAGE_MASK_F32_PADDED = 9 };
enum sage_status {
    SAGE_OK = 0,
    SAGE_E_INVALID = -1,     /* bad argument (shape, dtype, stride, null pointer) */
    SAGE_E_UNSUPPORTED = -2, /* valid for the reference but not built here (e.g. head_dim) */
    SAGE_E_LAUNCH = -3       /* the HIP runtime refused the launch */
};

/* A [B, H, L, D] tensor seen through strides (elements). */
typedef struct sage_tensor {
    void* ptr;
    int64_t stride_b, stride_h, stride_n;
} sage_tensor;

/*
 * Replaces the host function per_block_int8 and its two launches of
 * quant_per_block_int8_kernel (src/flag_attn/sage_attention/quant_per_block.py:49-101, kernel
 * :20-46), with the `k - km` pass (:53-54) fused into the K launch.
 *
 *   q, k         inputs, dtype in_dtype (SAGE_F16 / SAGE_BF16 / SAGE_F32)
 *   km           optional (ptr == NULL: none) K mean, dtype km_dtype, broadcast through its own
 *                strides (0 = broadcast); k - km is rounded once to diff_dtype exactly as the
 *                torch subtraction it replaces (the promoted dtype of k and km)
 *   q_int8,k_int8  outputs, int8, own strides
 *   q_scale      [B, Hq, ceil(M/blkq)] fp32 contiguous;  k_scale [B, Hkv, ceil(N/blkk)]
 *   q_mul        fp32 factor applied to Q before quantization (the reference passes
 *                sm_scale * 1.44269504 rounded to fp32); a value of exactly 1.0f multiplies nothing
 *   blkq, blkk   rows per quantization block (the attention kernel needs 128 / 64)
 * Either of q.ptr / k.ptr may be NULL to quantize only the other tensor.
 */
typedef struct sage_quant_params {
    sage_tensor q, k, km, q_int8, k_int8;
    float* q_scale;
    float* k_scale;
    int64_t batch, heads_q, heads_kv, qo_len, kv_len, head_dim;
    int32_t in_dtype, km_dtype, diff_dtype;
    int32_t blkq, blkk;
    float q_mul;
} sage_quant_params;

int sage_per_block_int8(const sage_quant_params* p, void* stream);

/*
 * Replaces the host function forward and its launch of _attn_fwd / _attn_fwd_inner
 * (src/flag_attn/sage_attention/attn_qk_int8_per_block.py:129-191, kernels :20-127).
 *
 *   q, k         int8 (per_block_int8 outputs), v: v_dtype (SAGE_F16 / SAGE_BF16)
 *   q_scale      [B, Hq, ceil(M/128)] fp32 contiguous;  k_scale [B, Hkv, ceil(N/64)]
 *   out          out_dtype (SAGE_F16 / SAGE_BF16 / SAGE_F32), own strides
 *   lse          optional [B, Hq, M] fp32 contiguous, base-2 log-sum-exp (:124-127); NULL = none
 *   mask         optional [B, Hq, M, N] through 4 strides (elements, 0 = broadcast);
 *                SAGE_MASK_BOOL: 1 byte per element, non-zero = keep, 0 = hide (:33-36,48), on every route;
 *                SAGE_MASK_BOOL_PADDED: the same, and the caller guarantees that every mask row can be read up to the
 *                next multiple of 16 bytes past kv_len and holds zeros there (a staging copy with padded rows): with
 *                16-byte aligned rows such a mask runs on the pipelined kernel for any kv_len, where a plain
 *                SAGE_MASK_BOOL needs kv_len % 16 == 0 for that;
 *                SAGE_MASK_BOOL_PADDED_CAUSAL: a padded mask of which the caller also guarantees mask[m, n] = 0 for
 *                n > m + (kv_len - qo_len) (the causal mask is folded in): the pipelined kernel then does not visit
 *                the key tiles beyond that limit, which the reference would skip one by one as all-False tiles;
 *                SAGE_MASK_F32 / SAGE_MASK_F16 / SAGE_MASK_BF16: additive, in that storage type (:38,50); masks with
 *                unit stride along the keys, 16-byte aligned rows and kv_len * entry size a multiple of 16 bytes (and
 *                no causal flag) run on the pipelined kernel, every other additive mask on the general one;
 *                SAGE_MASK_F16_PADDED / SAGE_MASK_BF16_PADDED / SAGE_MASK_F32_PADDED: the same, and the caller
 *                guarantees that every mask row can be read up to the next multiple of 16 bytes past kv_len (any finite
 *                values there): such a mask runs on the pipelined kernel for any kv_len
 *   causal       non-zero adds the bottom-right aligned causal mask n <= m + (N - M), handled
 *                like a bool mask (tiles that are entirely masked are skipped)
 * head_dim must be 64 or 128; heads_q must be a multiple of heads_kv.
 */
typedef struct sage_attn_params {
    sage_tensor q, k, v, out;
    const float* q_scale;
    const float* k_scale;
    float* lse;
    const void* mask;
    int64_t mask_stride_b, mask_stride_h, mask_stride_m, mask_stride_n;
    int64_t batch, heads_q, heads_kv, qo_len, kv_len, head_dim;
    int32_t v_dtype, out_dtype, mask_kind, causal;
} sage_attn_params;

int sage_attn_fwd(const sage_attn_params* p, void* stream);

/*
 * The same call with a workspace, for launches that would leave most of the chip idle: when
 * batch * heads_q * ceil(qo_len / 256) is well below the 256 compute units and no mask tensor is given, the keys
 * of every (batch, head, 256-query block) are cut into runs of whole 64-key steps, one workgroup each; the runs
 * write normalized fp32 partial outputs and their base-2 log-sum-exps to the workspace and a second kernel
 * combines them (out = sum_s 2^(lse_s - lse) o_s, lse = log2 sum_s 2^lse_s).  The reference's SageAttention
 * launch has no such split (attn_qk_int8_per_block.py:176-190 is one grid over q-blocks); its dense forward does
 * (see sage_flash_attn_fwd_ws).  Results agree with sage_attn_fwd to fp32 rounding of the combination.
 *   sage_attn_fwd_workspace_bytes  bytes the split of this call would use; 0 = the call would not split;
 *                                  -1 = invalid params (sage_hip_last_error says why)
 *   workspace                      device memory, 16-byte aligned, at least that large; NULL or smaller: no split,
 *                                  the call is sage_attn_fwd.  Contents need not be initialised and are not
 *                                  meaningful afterwards; calls on one stream may share one workspace.
 */
int64_t sage_attn_fwd_workspace_bytes(const sage_attn_params* p);
int sage_attn_fwd_ws(const sage_attn_params* p, void* workspace, int64_t workspace_bytes, void* stream);

/*
 * Mean of K over the sequence axis in a fixed fp32 order, for callers that want the library
 * to produce the `km` argument of per_block_int8 (the reference leaves km to its caller,
 * quant_per_block.py:49,53-54, so this entry point has no reference counterpart).
 * Order: 64-row chunks summed row by row from 0.0f; chunk partials summed in order from 0.0f;
 * total / (float)N; one rounding to out_dtype.  km_out: [B, Hkv, D] contiguous.
 * workspace: at least sage_k_mean_workspace_bytes(...) bytes of device memory, 16-byte aligned.
 */
int64_t sage_k_mean_workspace_bytes(int64_t batch, int64_t heads_kv, int64_t kv_len, int64_t head_dim);
int sage_k_mean(const sage_tensor* k, int32_t k_dtype, void* km_out, int32_t out_dtype, int64_t batch,
                int64_t heads_kv, int64_t kv_len, int64_t head_dim, void* workspace, void* stream);

/*
 * per_block_int8 with the K smoothing done by the library: km = sage_k_mean(k), then the quantization of
 * `k - km` and of q, as three launches instead of five (the Q blocks run side by side with the first pass over
 * K).  The reference leaves km to its caller (quant_per_block.py:49,53-54); its README's call sequence
 * (README.md:259-275: mean, per_block_int8, forward) is what this entry point stands for.  Results are
 * bit-identical to sage_k_mean followed by sage_per_block_int8 with that km.
 *
 *   quant        as for sage_per_block_int8; q and k share in_dtype; km / km_dtype / diff_dtype are ignored
 *                (the mean has k's dtype, so the difference is rounded to k's dtype); q.ptr may be NULL
 *   km_out       [B, Hkv, D] contiguous, in_dtype: the mean that was subtracted (required)
 *   q_dot_km     optional [B, Hq, M] fp32: sum over head_dim of fp32(q) * fp32(km of the row's KV head) — the
 *                amount by which smoothing lowers every logit q.k of that row before sm_scale, which a caller
 *                adds back to a log-sum-exp of the smoothed scores; NULL = not wanted
 *   workspace    sage_k_mean_workspace_bytes(batch, heads_kv, kv_len, head_dim) bytes, 16-byte aligned
 */
typedef struct sage_smooth_quant_params {
    sage_quant_params quant;
    void* km_out;
    float* q_dot_km;
    void* workspace;
} sage_smooth_quant_params;

int sage_per_block_int8_smooth_k(const sage_smooth_quant_params* p, void* stream);

/*
 * sage_k_mean without a workspace argument and without any allocation: no counterpart in the reference.
 * It is for callers that cannot allocate device memory around the call (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc): the chunk partials go to a fixed array inside the
 * library's device image, SAGE_K_MEAN_NOALLOC_MAX_WORKSPACE_BYTES per GPU, held until the process ends.
 * Same arguments, order of additions and result bits as sage_k_mean.  A call whose
 * sage_k_mean_workspace_bytes(...) exceeds the maximum is rejected with SAGE_E_UNSUPPORTED (nothing is
 * launched).  All calls on one GPU share that GPU's array: two calls that may run concurrently on one GPU
 * (different streams, different threads) race; calls ordered on one stream do not.  Nothing needs to start
 * from zero: every partial a call reads was written by that call.
 */
#define SAGE_K_MEAN_NOALLOC_MAX_WORKSPACE_BYTES (8 * 1024 * 1024)
int sage_k_mean_noalloc(const sage_tensor* k, int32_t k_dtype, void* km_out, int32_t out_dtype, int64_t batch,
                        int64_t heads_kv, int64_t kv_len, int64_t head_dim, void* stream);

/*
 * Dense attention forward on 16-bit Q, K, V: replaces the forward launch of FlagAttention's
 * flash_attention (src/flag_attn/flash.py:37-180 host, :346-510 kernel) for the calls that need no
 * dropout, no total attention and no gradient:  O = softmax(sm_scale * Q K^T [+ causal]) V.
 *
 *   q, k, v      dtype (SAGE_F16 / SAGE_BF16), own strides (any of the two layouts, GQA by heads_kv)
 *   out          out_dtype (SAGE_F16 / SAGE_BF16 / SAGE_F32), own strides
 *   log_normalizer  optional [B, Hq, M] fp32 contiguous: natural-log log-sum-exp of the scaled scores
 *                (flash.py:503-506); NULL = none
 *   causal       non-zero: key n is visible to query m iff n <= m + (N - M) (flash.py:53-54, P_SEQ);
 *                a query that sees no key (M > N) yields a zero row and a log normalizer of -inf
 *   sm_scale     factor on Q K^T (the host passes 1/sqrt(head_dim) by default, flash.py:57-58)
 * head_dim must be 64 or 128 (the reference also takes 16 and 32: a caller pads those with zero
 * channels, which changes neither Q K^T nor the first columns of P V); heads_q a multiple of heads_kv.
 */
typedef struct sage_flash_params {
    sage_tensor q, k, v, out;
    float* log_normalizer;
    int64_t batch, heads_q, heads_kv, qo_len, kv_len, head_dim;
    int32_t dtype, out_dtype, causal;
    float sm_scale;
} sage_flash_params;

int sage_flash_attn_fwd(const sage_flash_params* p, void* stream);

/*
 * The dense forward with the keys split over several workgroups where the launch would otherwise leave most of
 * the chip idle: replaces the split_kv branch of the reference's host function (src/flag_attn/flash.py:73-75,
 * :106-141: _fwd_split_kv_kernel into fp32 partials, then _fwd_combine_kv_splits; number of runs:
 * split_kv.py:250-278).  Workspace rules as for sage_attn_fwd_ws; the number of runs is chosen for 256 compute
 * units with 256-query workgroups, not by the reference's formula.
 */
int64_t sage_flash_attn_fwd_workspace_bytes(const sage_flash_params* p);
int sage_flash_attn_fwd_ws(const sage_flash_params* p, void* workspace, int64_t workspace_bytes, void* stream);

/*
 * The dense forward with dropout on P (src/flag_attn/flash.py:66-71 host side, :387-391, :467-502 kernel branch
 * IS_DROPOUT): element (b, h, m, n) of P survives iff
 *     rand(seed, offset + ((b * heads_q + h) * qo_len + m) * kv_len + n) > dropout_p
 * with Triton's tl.rand of six rounds (Philox-4x32 on the two words of the 64-bit offset, key = the two words of
 * the seed, first output word -> fp32 in [0, 1)); the softmax row sums and the log normalizer do not see the mask,
 * the output is scaled by 1 / (1 - dropout_p).  seed and offset are the caller's (the reference takes them from
 * torch's CUDA generator, dropout.py:17-28).  dropout_p in (0, 1); batch * heads_q * qo_len * kv_len < 2^31.
 * A plain kernel, an order of magnitude slower than sage_flash_attn_fwd: the generator dominates.
 *
 * sage_flash_dropout_mask writes the same mask on its own (src/flag_attn/testing/dropout.py:19-39):
 *   mask   [batch, heads_q, qo_len, kv_len] bytes, contiguous, 1 = kept
 */
int sage_flash_attn_fwd_dropout(const sage_flash_params* p, float dropout_p, uint64_t seed, uint64_t offset, void* stream);
int sage_flash_dropout_mask(uint8_t* mask, int64_t batch, int64_t heads_q, int64_t qo_len, int64_t kv_len,
                            float dropout_p, uint64_t seed, uint64_t offset, void* stream);

/*
 * Total attention of the same operator: total_attention[b, h, n] = sum over the queries m of
 * softmax(sm_scale * Q K^T [+ causal])[m, n], recomputed from Q, K and the log normalizer that
 * sage_flash_attn_fwd returned for the same arguments (src/flag_attn/total.py:22-160, called from
 * flash.py:142-157).  v, out and out_dtype of the params are not used.
 *   log_normalizer   [B, Hq, M] fp32 contiguous (natural log), as written by sage_flash_attn_fwd
 *   total_attention  [B, Hq, N] fp32 contiguous, written in full
 */
int sage_flash_total_attention(const sage_flash_params* p, const float* log_normalizer, float* total_attention,
                               void* stream);

/* Message describing the last non-zero status returned on this thread ("" if none). */
const char* sage_hip_last_error(void);

/* ABI version of this header; bumped when a struct layout changes. */
int sage_hip_abi_version(void);
#define SAGE_HIP_ABI_VERSION 3

#ifdef __cplusplus
}
#endif
#endif /* SAGE_ATTENTION_HIP_H */
