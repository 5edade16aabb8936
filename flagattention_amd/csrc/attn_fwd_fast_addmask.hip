// SageAttention forward for gfx950, pipelined kernel under an additive mask tensor stored as fp16, bf16 or fp32: the
// instances of attn_fast_kernel.h that stage mask entries of those types (FlagAttention
// src/flag_attn/sage_attention/attn_qk_int8_per_block.py:37-38,49-50: score + mask entry).  A translation unit of
// its own: twelve more instances of the kernel.
#include "attn_fast_kernel.h"

namespace sage {
namespace attn {
namespace {

template <int D, typename VT, typename MT>
int launch_additive(const AttnArgs& a, hipStream_t stream) {
    AttnArgs b = a;
    const int nq2 = (a.M + kFastRows - 1) / kFastRows;
    b.total_wg = (int)((int64_t)a.total_wg / a.nq * nq2);
    dim3 grid((unsigned)b.total_wg), block(kFastThreads);
    hipLaunchKernelGGL((sage_attn_fwd_fast_kernel<D, VT, true, 1, MT>), grid, block, 0, stream, b, nq2);
    return check_launch("sage_attn_fwd_fast_kernel (additive mask)");
}

template <int D, typename VT>
int launch_additive_mt(const AttnArgs& a, hipStream_t stream) {
    if (a.mask_dt == SAGE_F32) return launch_additive<D, VT, float>(a, stream);
    return a.mask_dt == SAGE_BF16 ? launch_additive<D, VT, __bf16>(a, stream) : launch_additive<D, VT, _Float16>(a, stream);
}

}  // namespace

int launch_fast_additive(const AttnArgs& a, int head_dim, int v_dtype, hipStream_t stream) {
    if (head_dim == 128)
        return v_dtype == SAGE_BF16 ? launch_additive_mt<128, __bf16>(a, stream) : launch_additive_mt<128, _Float16>(a, stream);
    return v_dtype == SAGE_BF16 ? launch_additive_mt<64, __bf16>(a, stream) : launch_additive_mt<64, _Float16>(a, stream);
}

}  // namespace attn
}  // namespace sage
