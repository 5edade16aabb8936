// SageAttention forward for gfx950, pipelined kernel: the int8 Q, K instances of attn_fast_kernel.h.
// They serve every call without a mask tensor (causal only with qo_len <= kv_len; any kv_len) and bool mask tensors
// with 16-byte aligned rows (padded by the caller where kv_len is not a multiple of 16), under the
// arithmetic contract of FlagAttention src/flag_attn/sage_attention/attn_qk_int8_per_block.py:20-127
// (per-block scales, base-2 online softmax, lse = log2(l) + m).
#include "attn_fast_kernel.h"

namespace sage {
namespace attn {
namespace {

template <int D, typename VT>
int launch_causal(const AttnArgs& a, bool causal, hipStream_t stream) {
    AttnArgs b = a;
    const int nq2 = (a.M + kFastRows - 1) / kFastRows;
    const int per_head = a.causal ? (nq2 + 1) / 2 : nq2;  // under the causal flag a workgroup takes two q-blocks
    b.total_wg = (int)((int64_t)a.total_wg / a.nq * per_head) * a.nsplit;
    dim3 grid((unsigned)b.total_wg), block(kFastThreads);
    if (causal) hipLaunchKernelGGL((sage_attn_fwd_fast_kernel<D, VT, true, 1>), grid, block, 0, stream, b, nq2);
    else hipLaunchKernelGGL((sage_attn_fwd_fast_kernel<D, VT, false, 1>), grid, block, 0, stream, b, nq2);
    return check_launch("sage_attn_fwd_fast_kernel");
}

template <int D, typename VT>
int launch_masked(const AttnArgs& a, hipStream_t stream) {
    AttnArgs b = a;
    const int nq2 = (a.M + kFastRows - 1) / kFastRows;
    b.total_wg = (int)((int64_t)a.total_wg / a.nq * nq2);
    dim3 grid((unsigned)b.total_wg), block(kFastThreads);
    hipLaunchKernelGGL((sage_attn_fwd_fast_kernel<D, VT, true, 1, bool>), grid, block, 0, stream, b, nq2);
    return check_launch("sage_attn_fwd_fast_kernel (bool mask)");
}

}  // namespace

// A bool mask tensor the pipelined kernel can stage with 16-byte loads: contiguous along the keys, every row start
// 16-byte aligned, no load that reaches past the end of a row (kv_len a multiple of 16, or rows that the caller
// padded with zeros to one), no causal flag on top.
// (esz: bytes per mask entry, 1 for bool masks, 2 / 4 for additive ones)
bool fast_serves_mask(const AttnArgs& a, int esz) {
    const int per16 = 16 / esz;  // entries per 16-byte load
    return a.mask != nullptr && !a.causal && a.ms_n == 1 && ((uintptr_t)a.mask % 16) == 0 &&
           a.ms_b % per16 == 0 && a.ms_h % per16 == 0 && a.ms_m % per16 == 0 && a.ms_m >= 0 && a.ms_m < (1 << 24) &&
           (a.N % per16 == 0 || a.mask_padded);
}

int launch_fast_masked(const AttnArgs& a, int head_dim, int v_dtype, hipStream_t stream) {
    if (a.mask_additive) return launch_fast_additive(a, head_dim, v_dtype, stream);
    if (head_dim == 128)
        return v_dtype == SAGE_BF16 ? launch_masked<128, __bf16>(a, stream) : launch_masked<128, _Float16>(a, stream);
    return v_dtype == SAGE_BF16 ? launch_masked<64, __bf16>(a, stream) : launch_masked<64, _Float16>(a, stream);
}

int launch_fast(const AttnArgs& a, int head_dim, int v_dtype, bool causal, hipStream_t stream) {
    causal = causal || (a.N % BN) != 0;  // the instance that can hide keys also serves a ragged last tile
    if (head_dim == 128)
        return v_dtype == SAGE_BF16 ? launch_causal<128, __bf16>(a, causal, stream)
                                    : launch_causal<128, _Float16>(a, causal, stream);
    return v_dtype == SAGE_BF16 ? launch_causal<64, __bf16>(a, causal, stream)
                                : launch_causal<64, _Float16>(a, causal, stream);
}

}  // namespace attn
}  // namespace sage
