// Dense attention forward with dropout on P for gfx950, and the dropout mask on its own
// (FlagAttention src/flag_attn/flash.py:387-391, :467-502 is the kernel branch it stands in for;
// src/flag_attn/testing/dropout.py:19-39 the helper that recomputes the mask).
//
// Element (b, h, m, n) of P survives iff rand(seed, offset + ((b H + h) M + m) N + n) > dropout_p, where rand is
// Triton's tl.rand with six rounds: Philox-4x32 on the counter (low word, high word, 0, 0) of the 64-bit sum,
// key (low, high) word of the seed, first output word x -> fp32 (x >= 0 ? x : -x - 1) * 4.6566127342e-10
// (x read as int32).  The row sums of the softmax are taken BEFORE the mask, the output is scaled by
// 1 / (1 - dropout_p) at the end (flash.py:470-477, :499-502).
//
// Six rounds of 32 x 32 -> 64 bit products per score cost an order of magnitude more than the softmax itself, so
// this kernel is a plain one, not the software-pipelined kernel of attn_fast_kernel.h: a wave owns 32 queries,
// walks over the keys 32 at a time, S^T = K Q^T and O^T += V^T P^T on v_mfma_f32_32x32x16 with K rows loaded
// straight into the A operand and V staged through LDS (two barriers per tile).
#include "attn_common.h"

namespace sage {
namespace {

using namespace attn;

// ---- Philox-4x32, six rounds, counter (c0, c1, 0, 0): the first output word
__device__ __forceinline__ uint32_t philox6_first_word(uint32_t c0, uint32_t c1, uint32_t k0, uint32_t k1) {
    constexpr uint32_t KEY_A = 0x9E3779B9u, KEY_B = 0xBB67AE85u, ROUND_A = 0xD2511F53u, ROUND_B = 0xCD9E8D57u;
    uint32_t c2 = 0, c3 = 0;
#pragma unroll
    for (int r = 0; r < 6; r++) {
        const uint64_t pb = (uint64_t)ROUND_B * c2, pa = (uint64_t)ROUND_A * c0;
        const uint32_t hi_b = (uint32_t)(pb >> 32), lo_b = (uint32_t)pb;
        const uint32_t hi_a = (uint32_t)(pa >> 32), lo_a = (uint32_t)pa;
        c0 = hi_b ^ c1 ^ k0;
        c2 = hi_a ^ c3 ^ k1;
        c1 = lo_b;
        c3 = lo_a;
        k0 += KEY_A;
        k1 += KEY_B;
    }
    return c0;
}

// does the element with this 64-bit offset survive?
__device__ __forceinline__ bool dropout_keeps(uint64_t offset, uint32_t k0, uint32_t k1, float dropout_p) {
    const int32_t x = (int32_t)philox6_first_word((uint32_t)offset, (uint32_t)(offset >> 32), k0, k1);
    const int32_t folded = x ^ (x >> 31);  // x >= 0 ? x : -x - 1
    return (float)folded * 4.6566127342e-10f > dropout_p;
}

struct DropArgs {
    const void* q;
    const void* k;
    const void* v;
    void* out;
    float* log_normalizer;  // [B, Hq, M] natural log, or null
    int64_t qs_b, qs_h, qs_n, ks_b, ks_h, ks_n, vs_b, vs_h, vs_n, os_b, os_h, os_n;
    int32_t Hq, M, N, groups, causal, out_dt;
    float qk_scale;    // sm_scale * log2(e)
    float dropout_p, keep_scale;  // keep_scale = 1 / (1 - dropout_p)
    uint32_t seed_lo, seed_hi;
    uint64_t offset;
};

constexpr int kDropWaves = 4;  // 128 queries per workgroup
constexpr int kDropKeys = 32;  // keys per tile

template <int D, typename VT>
__global__ __launch_bounds__(64 * kDropWaves) void flash_dropout_fwd_kernel(DropArgs a) {
    using PVT = PV<VT>;
    using vec16 = typename PVT::vec;
    constexpr int KS = D / 16;      // matrix instructions of one 32 x 32 score tile
    constexpr int DT = D / 32;      // 32-channel tiles of the output
    constexpr int V_RS = D + 2;     // LDS row stride in elements: rows four apart fall into different banks
    __shared__ VT vtile[kDropKeys * V_RS];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int l32 = lane & 31, half = lane >> 5;
    const int h = blockIdx.y, b = blockIdx.z, hk = h / a.groups;
    const int m0 = blockIdx.x * (32 * kDropWaves);
    const int my_m = m0 + 32 * wave + l32;
    const bool row_ok = my_m < a.M;
    const int shift = a.N - a.M;

    // Q rows as the B operand: lane (query l32, half) holds elements 16 t + 8 half .. + 7 of its row for step t
    vec16 qf[KS];
    {
        const VT* qp = static_cast<const VT*>(a.q) + (int64_t)b * a.qs_b + (int64_t)h * a.qs_h +
                       (int64_t)min(my_m, a.M - 1) * a.qs_n + 8 * half;
#pragma unroll
        for (int t = 0; t < KS; t++) qf[t] = *reinterpret_cast<const vec16*>(qp + 16 * t);
    }
    const VT* kbase = static_cast<const VT*>(a.k) + (int64_t)b * a.ks_b + (int64_t)hk * a.ks_h + 8 * half;
    const VT* vbase = static_cast<const VT*>(a.v) + (int64_t)b * a.vs_b + (int64_t)hk * a.vs_h;
    // offset of element (b, h, my_m, 0) in the random stream
    const uint64_t rng_row = a.offset + (((uint64_t)b * a.Hq + h) * (uint64_t)a.M + (uint64_t)my_m) * (uint64_t)a.N;

    // keys that any row of the workgroup can see
    int n_end = a.N;
    if (a.causal) n_end = max(min(a.N, min(m0 + 32 * kDropWaves, a.M) + shift), 0);
    const int my_lim = a.causal ? min(my_m + shift, a.N - 1) : a.N - 1;  // last key this lane's query sees

    v16f acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[dt][i] = 0.0f;
    float m_i = -INFINITY, l_i = 0.0f;  // running maximum (base-2 units) and this half's part of the row sum

    for (int n0 = 0; n0 < n_end; n0 += kDropKeys) {
        // K rows as the A operand: lane (key l32, half); rows past the end re-read the last one (their scores are hidden)
        vec16 kf[KS];
        {
            const VT* kp = kbase + (int64_t)min(n0 + l32, a.N - 1) * a.ks_n;
#pragma unroll
            for (int t = 0; t < KS; t++) kf[t] = *reinterpret_cast<const vec16*>(kp + 16 * t);
        }
        // V tile -> LDS, 16 bytes per thread and round
        __syncthreads();  // the previous tile has been read
#pragma unroll
        for (int c = threadIdx.x; c < kDropKeys * D / 8; c += 64 * kDropWaves) {
            const int row = c / (D / 8), piece = c % (D / 8);
            const vec16 x = *reinterpret_cast<const vec16*>(vbase + (int64_t)min(n0 + row, a.N - 1) * a.vs_n + 8 * piece);
            // (rows are 4-byte aligned only: V_RS is not a multiple of 8 elements)
            typedef uint32_t __attribute__((may_alias)) word;
            word w[4];
            __builtin_memcpy(w, &x, 16);
            word* dst = reinterpret_cast<word*>(&vtile[row * V_RS + 8 * piece]);
#pragma unroll
            for (int j = 0; j < 4; j++) dst[j] = w[j];
        }
        __syncthreads();

        v16f s;
#pragma unroll
        for (int i = 0; i < 16; i++) s[i] = 0.0f;
#pragma unroll
        for (int t = 0; t < KS; t++) s = PVT::mfma(kf[t], qf[t], s);

        // accumulator i of this lane: key n0 + 8 (i / 4) + 4 half + i % 4 of query my_m
        float tile_max = -INFINITY;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int n = n0 + 8 * (i >> 2) + 4 * half + (i & 3);
            s[i] = n <= my_lim ? s[i] * a.qk_scale : -INFINITY;
            tile_max = fmaxf(tile_max, s[i]);
        }
        tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32));
        const float m_new = fmaxf(m_i, tile_max);
        // (a query that has seen no key yet keeps m = -inf: every p below is then 0 and alpha is 1)
        const float m_use = m_new == -INFINITY ? 0.0f : m_new;
        const float alpha = m_i == -INFINITY ? 1.0f : __builtin_amdgcn_exp2f(m_i - m_use);
        float psum = 0.0f;
        vec16 pf[2];
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int n = n0 + 8 * (i >> 2) + 4 * half + (i & 3);
            float p = __builtin_amdgcn_exp2f(s[i] - m_use);  // hidden keys: exp2(-inf) = 0
            psum += p;                                        // the row sum does not see the dropout mask
            if (!dropout_keeps(rng_row + (uint64_t)n, a.seed_lo, a.seed_hi, a.dropout_p)) p = 0.0f;
            pf[i >> 3][i & 7] = (VT)p;
        }
        l_i = l_i * alpha + psum;
        m_i = m_new;
#pragma unroll
        for (int dt = 0; dt < DT; dt++) {
#pragma unroll
            for (int i = 0; i < 16; i++) acc[dt][i] *= alpha;
#pragma unroll
            for (int t = 0; t < 2; t++) {
                // V^T as the A operand, in the key order of pf[t]: element j is key 16 t + 8 (j / 4) + 4 half + j % 4
                vec16 vf;
#pragma unroll
                for (int j = 0; j < 8; j++)
                    vf[j] = vtile[(16 * t + 8 * (j >> 2) + 4 * half + (j & 3)) * V_RS + 32 * dt + l32];
                acc[dt] = PVT::mfma(vf, pf[t], acc[dt]);
            }
        }
    }

    const float l_tot = l_i + __shfl_xor(l_i, 32);
    const float inv = l_tot > 0.0f ? a.keep_scale / l_tot : 0.0f;  // l = 0: a query that saw no key: zero row
    if (!row_ok) return;
    // accumulator i of tile dt: channel 32 dt + 8 (i / 4) + 4 half + i % 4 of query my_m
    const int64_t obase = (int64_t)b * a.os_b + (int64_t)h * a.os_h + (int64_t)my_m * a.os_n;
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const int d = 32 * dt + 8 * g + 4 * half;
            float r[4];
#pragma unroll
            for (int i = 0; i < 4; i++) r[i] = acc[dt][4 * g + i] * inv;
            if (a.out_dt == SAGE_BF16) {
                typedef __bf16 b4 __attribute__((ext_vector_type(4)));
                *reinterpret_cast<b4*>(static_cast<__bf16*>(a.out) + obase + d) = b4{(__bf16)r[0], (__bf16)r[1], (__bf16)r[2], (__bf16)r[3]};
            } else if (a.out_dt == SAGE_F16) {
                typedef _Float16 h4 __attribute__((ext_vector_type(4)));
                *reinterpret_cast<h4*>(static_cast<_Float16*>(a.out) + obase + d) = h4{(_Float16)r[0], (_Float16)r[1], (_Float16)r[2], (_Float16)r[3]};
            } else {
                *reinterpret_cast<v4f*>(static_cast<float*>(a.out) + obase + d) = v4f{r[0], r[1], r[2], r[3]};
            }
        }
    if (a.log_normalizer && half == 0)
        a.log_normalizer[((int64_t)b * a.Hq + h) * a.M + my_m] =
            l_tot > 0.0f ? (__builtin_log2f(l_tot) + m_i) * 0.693147180559945309f : -INFINITY;
}

__global__ void dropout_mask_kernel(uint8_t* mask, int64_t count, uint64_t offset, uint32_t seed_lo, uint32_t seed_hi,
                                    float dropout_p) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) mask[i] = dropout_keeps(offset + (uint64_t)i, seed_lo, seed_hi, dropout_p) ? 1 : 0;
}

template <int D, typename VT>
int launch_drop(const DropArgs& a, int64_t B, hipStream_t stream) {
    dim3 grid((unsigned)((a.M + 32 * kDropWaves - 1) / (32 * kDropWaves)), (unsigned)a.Hq, (unsigned)B), block(64 * kDropWaves);
    hipLaunchKernelGGL((flash_dropout_fwd_kernel<D, VT>), grid, block, 0, stream, a);
    return check_launch("flash_dropout_fwd_kernel");
}

}  // namespace

int launch_flash_dropout(const sage_flash_params& p, float dropout_p, uint64_t seed, uint64_t offset, hipStream_t stream) {
    DropArgs a{};
    a.q = p.q.ptr; a.k = p.k.ptr; a.v = p.v.ptr; a.out = p.out.ptr; a.log_normalizer = p.log_normalizer;
    a.qs_b = p.q.stride_b; a.qs_h = p.q.stride_h; a.qs_n = p.q.stride_n;
    a.ks_b = p.k.stride_b; a.ks_h = p.k.stride_h; a.ks_n = p.k.stride_n;
    a.vs_b = p.v.stride_b; a.vs_h = p.v.stride_h; a.vs_n = p.v.stride_n;
    a.os_b = p.out.stride_b; a.os_h = p.out.stride_h; a.os_n = p.out.stride_n;
    a.Hq = (int)p.heads_q; a.M = (int)p.qo_len; a.N = (int)p.kv_len; a.groups = (int)(p.heads_q / p.heads_kv);
    a.causal = p.causal ? 1 : 0; a.out_dt = p.out_dtype;
    a.qk_scale = p.sm_scale * 1.44269504089f;
    a.dropout_p = dropout_p;
    a.keep_scale = 1.0f / (1.0f - dropout_p);
    a.seed_lo = (uint32_t)seed; a.seed_hi = (uint32_t)(seed >> 32);
    a.offset = offset;
    if (p.heads_q > 65535 || p.batch > 65535)
        return fail(SAGE_E_UNSUPPORTED, "sage_flash_attn_fwd_dropout: more than 65535 heads or batches");
    if (p.head_dim == 128)
        return p.dtype == SAGE_BF16 ? launch_drop<128, __bf16>(a, p.batch, stream) : launch_drop<128, _Float16>(a, p.batch, stream);
    return p.dtype == SAGE_BF16 ? launch_drop<64, __bf16>(a, p.batch, stream) : launch_drop<64, _Float16>(a, p.batch, stream);
}

int launch_dropout_mask(uint8_t* mask, int64_t count, float dropout_p, uint64_t seed, uint64_t offset, hipStream_t stream) {
    if (count == 0) return SAGE_OK;
    const int64_t blocks = (count + 255) / 256;
    if (blocks > 0x7fffffffLL) return fail(SAGE_E_UNSUPPORTED, "sage_flash_dropout_mask: too many elements for one launch");
    hipLaunchKernelGGL(dropout_mask_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, mask, count, offset,
                       (uint32_t)seed, (uint32_t)(seed >> 32), dropout_p);
    return check_launch("dropout_mask_kernel");
}

}  // namespace sage
