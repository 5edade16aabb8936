// SageAttention forward for gfx950, pipelined kernel: the int8 Q, K instances of attn_fast_kernel.h.
// They serve every call without a mask tensor (causal only with qo_len <= kv_len; any kv_len), under the
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
    b.total_wg = (int)((int64_t)a.total_wg / a.nq * per_head);
    dim3 grid((unsigned)b.total_wg), block(kFastThreads);
    if (causal) hipLaunchKernelGGL((sage_attn_fwd_fast_kernel<D, VT, true, 1>), grid, block, 0, stream, b, nq2);
    else hipLaunchKernelGGL((sage_attn_fwd_fast_kernel<D, VT, false, 1>), grid, block, 0, stream, b, nq2);
    return check_launch("sage_attn_fwd_fast_kernel");
}

}  // namespace

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
