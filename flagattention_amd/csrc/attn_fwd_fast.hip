// Software-pipelined SageAttention forward for gfx950: every call without a mask tensor (causal
// only with qo_len <= kv_len; any kv_len).  Same arithmetic contract as the general
// kernel in attn_fwd.hip (FlagAttention src/flag_attn/sage_attention/attn_qk_int8_per_block.py:
// 20-127); what differs is how the work is laid out in time.
//
// Per workgroup: 8 waves x 32 query rows (two q_scale blocks, so that every K/V tile staged in LDS
// serves 256 rows); per step: 64 keys.  Every wave computes the transposed
// products S^T = K.Q^T (8 x v_mfma_i32_32x32x32_i8) and O^T += V^T.P^T (16 x v_mfma_f32_32x32x16)
// so that a lane owns one query row and P never leaves registers.
//
// * K and V tiles go from global memory straight into LDS (global_load_lds_dwordx4, 16 bytes per
//   lane), four tiles of each resident: tile t lives in buffer t % 4 and is fetched during the VALU
//   phase two (V) or three (K) steps before the step that multiplies with it.  LDS rows are
//   unpadded; bank conflicts are avoided by an XOR swizzle of the 16-byte chunks of a row, applied
//   on the global-address side of the load and undone by the fragment reads.
// * V is read with ds_read_b64_tr_b16, which hands each lane four consecutive keys of one channel:
//   exactly the A operand of the P.V MFMA, with no shuffling instructions.
// * Every wave alternates between a VALU phase (exponentials of step j) and an MFMA phase (Q.K^T of
//   step j+1 and P.V of step j back to back, with the row sums of P riding in the shadow of the
//   matrix instructions).  The two waves that share a SIMD
//   run half a step apart, so the matrix core and the VALU are both kept busy; phases are
//   separated by workgroup barriers (two per step).
// * The int32 Q.K^T accumulators start from the bit pattern of 1.5 * 2^23, so their bits ARE the
//   float kBias + dot and no int -> float conversion is issued; the two score register sets swap
//   roles every step (the loop body exists for both parities).
// * No row maximum is taken per step: exponentials use the reference point the row already has
//   (the maximum of its first tile to begin with), and a step whose row sums come out large is
//   redone against its true maximum before any P.V instruction of it has been issued.  The row
//   sums are needed anyway, so the common step pays nothing for the check but a compare.
// * 16-bit outputs are transposed through LDS and written as whole rows.
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
