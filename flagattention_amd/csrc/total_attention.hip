// Total attention of the dense flash_attention for gfx950: tot[b, h, n] = sum over queries m of
// softmax(sm_scale * q.k^T)[m, n], recomputed from Q, K and the log normalizer the forward pass returned
// (FlagAttention src/flag_attn/total.py:64-160 is the kernel it stands in for, flash.py:142-157 its call site).
//
// One wave owns 32 keys for the whole launch and walks over the queries 32 at a time:
//   S^T[key, query] = K . Q^T   (v_mfma_f32_32x32x16_{bf16,f16}: A = the wave's K rows, kept in registers;
//                                B = the query rows, each lane loading the 16-byte pieces of its own row)
//   p = exp2(S^T * sm_scale * log2(e) - L[query] * log2(e)),   zero where the causal mask hides the key.
// A lane owns one query column of every tile and sixteen of the 32 keys, so the sum over queries is first kept
// per lane (sixteen running sums) and folded across the 32 lanes of each half of the wave once, at the end.
// No LDS, no barriers; the next tile's query pieces are requested before the current tile is multiplied.
#include "attn_common.h"

namespace sage {
namespace {

using namespace attn;

struct TotalArgs {
    const void* q;
    const void* k;
    const float* log_normalizer;  // [B, Hq, M], natural log
    float* total;                 // [B, Hq, N]
    int64_t qs_b, qs_h, qs_n;
    int64_t ks_b, ks_h, ks_n;
    int32_t Hq, M, N, groups, causal;
    float qk_scale;  // sm_scale * log2(e)
};

constexpr int kTotalWaves = 4;  // 128 keys per workgroup

template <int D, typename VT>
__global__ __launch_bounds__(64 * kTotalWaves) void total_attention_kernel(TotalArgs a) {
    using PVT = PV<VT>;
    using vec16 = typename PVT::vec;
    constexpr int KS = D / 16;  // matrix instructions per 32 x 32 tile
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int l32 = lane & 31, half = lane >> 5;
    const int h = blockIdx.y, b = blockIdx.z;
    const int n0 = (blockIdx.x * kTotalWaves + wave) * 32;
    if (n0 >= a.N) return;  // (no barrier in this kernel)
    const int hk = h / a.groups;
    const int shift = a.N - a.M;

    // K rows of this wave: lane (key l32, half) holds elements 16 t + 8 half .. + 7 of its row for step t
    vec16 kf[KS];
    {
        const int key = min(n0 + l32, a.N - 1);  // keys past the end re-read the last one; their sums are not stored
        const VT* kp = static_cast<const VT*>(a.k) + (int64_t)b * a.ks_b + (int64_t)hk * a.ks_h + (int64_t)key * a.ks_n + 8 * half;
#pragma unroll
        for (int t = 0; t < KS; t++) kf[t] = *reinterpret_cast<const vec16*>(kp + 16 * t);
    }
    const VT* qbase = static_cast<const VT*>(a.q) + (int64_t)b * a.qs_b + (int64_t)h * a.qs_h + 8 * half;
    const float* lbase = a.log_normalizer + ((int64_t)b * a.Hq + h) * a.M;

    // queries that can see any of this wave's keys: m + shift >= n0
    int m_lo = 0;
    if (a.causal) m_lo = (max(n0 - shift, 0) / 32) * 32;
    float tot[16];
#pragma unroll
    for (int i = 0; i < 16; i++) tot[i] = 0.0f;

    auto load_tile = [&](int m0, vec16 (&qf)[KS], float& lq) {
        const int m = min(m0 + l32, a.M - 1);
        const VT* qp = qbase + (int64_t)m * a.qs_n;
#pragma unroll
        for (int t = 0; t < KS; t++) qf[t] = *reinterpret_cast<const vec16*>(qp + 16 * t);
        lq = lbase[m] * 1.44269504088896340736f;
    };
    vec16 qf[2][KS];
    float lq[2];
    if (m_lo < a.M) load_tile(m_lo, qf[0], lq[0]);
    int buf = 0;
    for (int m0 = m_lo; m0 < a.M; m0 += 32, buf ^= 1) {
        if (m0 + 32 < a.M) {
            if (buf == 0) load_tile(m0 + 32, qf[1], lq[1]);
            else load_tile(m0 + 32, qf[0], lq[0]);
        }
        v16f s;
#pragma unroll
        for (int i = 0; i < 16; i++) s[i] = 0.0f;
        if (buf == 0) {
#pragma unroll
            for (int t = 0; t < KS; t++) s = PVT::mfma(kf[t], qf[0][t], s);
        } else {
#pragma unroll
            for (int t = 0; t < KS; t++) s = PVT::mfma(kf[t], qf[1][t], s);
        }
        const float l2 = buf == 0 ? lq[0] : lq[1];
        const int m = m0 + l32;
        const bool row_ok = m < a.M;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int n = n0 + 8 * (i >> 2) + 4 * half + (i & 3);  // key of accumulator register i in this lane
            const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(s[i], a.qk_scale, -l2));
            const bool seen = row_ok && (!a.causal || n <= m + shift);
            tot[i] += seen ? p : 0.0f;  // (a select, not a product: a query that sees no key has L = -inf, p = inf)
        }
    }
    // fold the 32 query columns of each half
#pragma unroll
    for (int i = 0; i < 16; i++) {
        float x = tot[i];
#pragma unroll
        for (int off = 16; off > 0; off >>= 1) x += __shfl_xor(x, off);
        tot[i] = x;
    }
    if (l32 == 0) {
        float* out = a.total + ((int64_t)b * a.Hq + h) * a.N;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int n = n0 + 8 * (i >> 2) + 4 * half + (i & 3);
            if (n < a.N) out[n] = tot[i];
        }
    }
}

template <int D, typename VT>
int launch_total(const TotalArgs& a, int64_t B, hipStream_t stream) {
    dim3 grid((unsigned)((a.N + 32 * kTotalWaves - 1) / (32 * kTotalWaves)), (unsigned)a.Hq, (unsigned)B), block(64 * kTotalWaves);
    hipLaunchKernelGGL((total_attention_kernel<D, VT>), grid, block, 0, stream, a);
    return check_launch("total_attention_kernel");
}

}  // namespace

int launch_flash_total_attention(const sage_flash_params& p, const float* log_normalizer, float* total, hipStream_t stream) {
    TotalArgs a{};
    a.q = p.q.ptr; a.k = p.k.ptr; a.log_normalizer = log_normalizer; a.total = total;
    a.qs_b = p.q.stride_b; a.qs_h = p.q.stride_h; a.qs_n = p.q.stride_n;
    a.ks_b = p.k.stride_b; a.ks_h = p.k.stride_h; a.ks_n = p.k.stride_n;
    a.Hq = (int)p.heads_q; a.M = (int)p.qo_len; a.N = (int)p.kv_len; a.groups = (int)(p.heads_q / p.heads_kv);
    a.causal = p.causal ? 1 : 0;
    a.qk_scale = p.sm_scale * 1.44269504089f;
    if (p.heads_q > 65535 || p.batch > 65535) return fail(SAGE_E_UNSUPPORTED, "sage_flash_total_attention: more than 65535 heads or batches");
    if (p.head_dim == 128)
        return p.dtype == SAGE_BF16 ? launch_total<128, __bf16>(a, p.batch, stream) : launch_total<128, _Float16>(a, p.batch, stream);
    return p.dtype == SAGE_BF16 ? launch_total<64, __bf16>(a, p.batch, stream) : launch_total<64, _Float16>(a, p.batch, stream);
}

}  // namespace sage
