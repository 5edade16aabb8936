// SageAttention forward for gfx950 (MI355X): INT8 Q.K^T on MFMA with int32 accumulation,
// block-scale dequantization, fp32 online softmax (base 2), 16-bit P.V on MFMA.
//
// Replaces _attn_fwd / _attn_fwd_inner of FlagAttention
// (src/flag_attn/sage_attention/attn_qk_int8_per_block.py:20-127).  Semantics kept: one q_scale
// per 128 query rows and one k_scale per 64 keys (:42,115), scores = fp32(int32 dot) *
// (q_scale * k_scale) (:44), masked / out-of-range scores get -1e6 added (:38,48,52), a 128x64
// tile whose bool mask is False everywhere is skipped (:33-36), rows start at m = -inf, l = 1
// (:110-111), lse = log2(l) + m (:126).
//
// Work decomposition (wave64, 32x32 MFMA tiles):
//   workgroup = 4 waves = 128 query rows (one q_scale); wave w owns rows 32w .. 32w+31.
//   Each KV step covers 64 keys (one k_scale).  The transposed products are computed,
//       S^T[kv, q] = K . Q^T   (v_mfma_i32_32x32x32_i8,  A = K rows,   B = Q rows)
//       O^T[d,  q] = V^T . P^T (v_mfma_f32_32x32x16_*,   A = V^T rows, B = P^T)
//   so that every lane owns ONE query row (column q = lane % 32 of each accumulator tile): row
//   max / row sum / alpha / q_scale are per-lane scalars, and the S^T accumulator registers are
//   already laid out as the B operand of the P.V product (P never leaves registers).  The kv
//   order inside an MFMA k-step is free as long as both operands agree; V^T is staged in LDS in
//   exactly the order the S^T accumulator layout dictates (see v_chunk()).
//   K tiles (int8 [64][D]) and V tiles (16-bit, transposed to [D][64]) are double buffered in LDS;
//   global loads for step j+1 are issued before the math of step j.
#include "attn_common.h"

namespace sage {
using namespace attn;
namespace {

template <int D>
struct Tile {
    static constexpr int KSTEPS = D / 32;           // int8 MFMA k-steps over head_dim
    static constexpr int DTILES = D / 32;           // 32-row tiles of O^T
    static constexpr int K_RS = D + 16;             // K tile row stride (bytes); +16 spreads rows over banks
    static constexpr int K_BYTES = BN * K_RS;
    static constexpr int V_RS = BN * 2;             // V^T row stride (bytes), XOR-swizzled 16-byte chunks
    static constexpr int V_BYTES = D * V_RS;
    static constexpr int STAGE = K_BYTES + V_BYTES;
    static constexpr int K_CHUNKS_PER_ROW = D / 16;
    static constexpr int K_LOADS = BN * K_CHUNKS_PER_ROW / kThreads;  // 16-byte loads per thread per K tile
    static constexpr int V_ITEMS = (D / 8) * (BN / 4);                 // (8 channels x 4 keys) items per V tile
};

// XOR swizzle of the 16-byte chunk index inside a V^T row (row = channel d).
__device__ __forceinline__ int v_swz(int d) { return (d ^ (d >> 3)) & 7; }

// Chunk (16 bytes = 8 keys) and half-chunk (4 consecutive keys) that the run of keys
// [4r, 4r+4) of a 64-key tile occupies in a V^T row.  The order is the one in which the S^T
// accumulator hands P to the P.V MFMA: lane half h, k-step t' (16 keys each), slot c of 8 holds
// key 16t' + 8(c/4) + 4h + c%4, i.e. run r = 4t' + 2(c/4) + h  ->  chunk 2t' + h, half c/4.
__device__ __forceinline__ int v_chunk(int r) { return ((r >> 2) << 1) | (r & 1); }
__device__ __forceinline__ int v_halfchunk(int r) { return (r >> 1) & 1; }

__device__ __forceinline__ float xhalf_max(float x) { return fmaxf(x, __shfl_xor(x, 32)); }
__device__ __forceinline__ float xhalf_sum(float x) {
    const float o = __shfl_xor(x, 32);
    return (threadIdx.x & 32) ? (o + x) : (x + o);  // same operand order in both halves
}

// Additive mask entries as fp32, whatever the mask's storage type (fp32, fp16 or bf16: a.mask_dt).
__device__ __forceinline__ float mask_entry(const AttnArgs& a, int64_t idx) {
    if (a.mask_dt == SAGE_F32) return static_cast<const float*>(a.mask)[idx];
    if (a.mask_dt == SAGE_BF16) return (float)static_cast<const __bf16*>(a.mask)[idx];
    return (float)static_cast<const _Float16*>(a.mask)[idx];
}
__device__ __forceinline__ float4 mask_run4(const AttnArgs& a, int64_t idx) {  // four consecutive, naturally aligned entries
    if (a.mask_dt == SAGE_F32) return *reinterpret_cast<const float4*>(static_cast<const float*>(a.mask) + idx);
    const uint2 w = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(a.mask) + idx);
    if (a.mask_dt == SAGE_BF16)
        return make_float4(__builtin_bit_cast(float, w.x << 16), __builtin_bit_cast(float, w.x & 0xffff0000u),
                           __builtin_bit_cast(float, w.y << 16), __builtin_bit_cast(float, w.y & 0xffff0000u));
    return make_float4((float)__builtin_bit_cast(_Float16, (uint16_t)(w.x & 0xffffu)), (float)__builtin_bit_cast(_Float16, (uint16_t)(w.x >> 16)),
                       (float)__builtin_bit_cast(_Float16, (uint16_t)(w.y & 0xffffu)), (float)__builtin_bit_cast(_Float16, (uint16_t)(w.y >> 16)));
}

template <int D, typename VT, int MODE>
__global__ __launch_bounds__(kThreads, 2) void sage_attn_fwd_kernel(AttnArgs a) {
    using T = Tile<D>;
    using PVT = PV<VT>;
    using vec16 = typename PVT::vec;
    __shared__ __attribute__((aligned(16))) unsigned char smem[2 * T::STAGE];

    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int l32 = lane & 31;
    const int half = lane >> 5;

    // Workgroup -> (batch, head, q-block).  Consecutive workgroup ids land on different XCDs
    // (8 of them, round robin); remap so that each XCD walks a contiguous range of logical ids and
    // therefore keeps one head's K/V in its own L2 while it sweeps that head's q-blocks.
    int wg = blockIdx.x;
    {
        const int per_xcd = a.total_wg >> 3;
        if ((a.total_wg & 7) == 0) wg = (wg & 7) * per_xcd + (wg >> 3);
    }
    const int ht = MODE >= MODE_MASK_BOOL ? a.head_tile : 1;  // heads that alternate within a q-block (shared mask)
    int iq = (wg / ht) % a.nq;
    if (MODE == MODE_CAUSAL) iq = a.nq - 1 - iq;  // longest rows first
    const int h = (wg / (ht * a.nq)) % (a.Hq / ht) * ht + wg % ht;
    const int b = wg / (a.nq * a.Hq);
    const int hk = h / a.groups;
    const int m0 = iq * BM;
    const int my_m = m0 + 32 * wave + l32;
    const bool row_ok = my_m < a.M;

    // ---- Q fragments (B operand of S^T = K.Q^T): lane (q = l32, half) holds channels
    //      half*D/2 + 16t .. +15 for k-step t.  K fragments use the same channel order.
    v4i qf[T::KSTEPS];
    {
        const int8_t* qp = a.q + (int64_t)b * a.qs_b + (int64_t)h * a.qs_h + (int64_t)my_m * a.qs_n + half * (D / 2);
#pragma unroll
        for (int t = 0; t < T::KSTEPS; t++)
            qf[t] = row_ok ? *reinterpret_cast<const v4i*>(qp + 16 * t) : v4i{0, 0, 0, 0};
    }
    const float qs = a.q_scale[((int64_t)b * a.Hq + h) * a.nq + iq];
    const float* ksp = a.k_scale + ((int64_t)b * a.Hkv + hk) * a.nk;

    // ---- number of KV steps
    int nsteps = a.nk;
    if (MODE == MODE_CAUSAL || (MODE >= MODE_MASK_BOOL && a.causal)) {
        // last visible column of the last valid row of this q-block
        const int last_row = min(m0 + BM, a.M) - 1;
        const int64_t hi = (int64_t)last_row + (a.N - a.M) + 1;  // exclusive
        const int64_t hic = hi < (int64_t)a.N ? hi : (int64_t)a.N;
        const int vis = hi <= 0 ? 0 : (int)((hic + BN - 1) / BN);
        nsteps = min(nsteps, vis);
    }

    // ---- staging roles
    const int8_t* kg = a.k + (int64_t)b * a.ks_b + (int64_t)hk * a.ks_h;
    const VT* vg = static_cast<const VT*>(a.v) + (int64_t)b * a.vs_b + (int64_t)hk * a.vs_h;
    int k_row[T::K_LOADS], k_lds[T::K_LOADS], k_col[T::K_LOADS], k_off[T::K_LOADS];
#pragma unroll
    for (int j = 0; j < T::K_LOADS; j++) {
        const int id = tid + kThreads * j;
        k_row[j] = id / T::K_CHUNKS_PER_ROW;
        k_col[j] = 16 * (id % T::K_CHUNKS_PER_ROW);
        k_lds[j] = k_row[j] * T::K_RS + k_col[j];
        k_off[j] = k_row[j] * (int)a.ks_n + k_col[j];  // byte offset inside a tile (host checks it fits 31 bits)
    }
    const bool v_worker = tid < T::V_ITEMS;
    const int v_dg = tid % (D / 8);  // group of 8 channels
    const int v_r = tid / (D / 8);   // run of 4 keys
    int v_lds[8], v_off[4];
#pragma unroll
    for (int e = 0; e < 8; e++) {
        const int d = 8 * v_dg + e;
        v_lds[e] = T::K_BYTES + d * T::V_RS + ((v_chunk(v_r) ^ v_swz(d)) * 16) + v_halfchunk(v_r) * 8;
    }
#pragma unroll
    for (int i = 0; i < 4; i++) v_off[i] = (4 * v_r + i) * (int)a.vs_n + 8 * v_dg;  // element offset inside a tile

    v4i kreg[T::K_LOADS];
    uint4 vreg[4];
    auto load_tile = [&](int step) {
        const int n0 = step * BN;
        const int8_t* kt = kg + (int64_t)n0 * a.ks_n;  // uniform tile bases, 32-bit per-lane offsets
        const VT* vt = vg + (int64_t)n0 * a.vs_n;
        if (n0 + BN <= a.N) {
#pragma unroll
            for (int j = 0; j < T::K_LOADS; j++) kreg[j] = *reinterpret_cast<const v4i*>(kt + k_off[j]);
            if (v_worker) {
#pragma unroll
                for (int i = 0; i < 4; i++) vreg[i] = *reinterpret_cast<const uint4*>(vt + v_off[i]);
            }
        } else {
            // last, partial tile: keys past N read as zeros (their scores get -1e6, their V rows weigh 0)
            const int last = a.N - 1 - n0;
#pragma unroll
            for (int j = 0; j < T::K_LOADS; j++) {
                const int r = min(k_row[j], last);
                kreg[j] = *reinterpret_cast<const v4i*>(kt + (int64_t)r * a.ks_n + k_col[j]);
                if (k_row[j] > last) kreg[j] = v4i{0, 0, 0, 0};
            }
            if (v_worker) {
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int r = min(4 * v_r + i, last);
                    vreg[i] = *reinterpret_cast<const uint4*>(vt + (int64_t)r * a.vs_n + 8 * v_dg);
                    if (4 * v_r + i > last) vreg[i] = make_uint4(0, 0, 0, 0);
                }
            }
        }
    };
    auto store_tile = [&](int buf) {
        unsigned char* base = smem + buf * T::STAGE;
#pragma unroll
        for (int j = 0; j < T::K_LOADS; j++) *reinterpret_cast<v4i*>(base + k_lds[j]) = kreg[j];
        if (v_worker) {
            const uint32_t r0[4] = {vreg[0].x, vreg[0].y, vreg[0].z, vreg[0].w};
            const uint32_t r1[4] = {vreg[1].x, vreg[1].y, vreg[1].z, vreg[1].w};
            const uint32_t r2[4] = {vreg[2].x, vreg[2].y, vreg[2].z, vreg[2].w};
            const uint32_t r3[4] = {vreg[3].x, vreg[3].y, vreg[3].z, vreg[3].w};
#pragma unroll
            for (int i = 0; i < 4; i++) {
                // channel 2i (low halves) and 2i+1 (high halves) of four consecutive keys
                uint2 lo, hi;
                lo.x = __builtin_amdgcn_perm(r1[i], r0[i], 0x05040100u);
                lo.y = __builtin_amdgcn_perm(r3[i], r2[i], 0x05040100u);
                hi.x = __builtin_amdgcn_perm(r1[i], r0[i], 0x07060302u);
                hi.y = __builtin_amdgcn_perm(r3[i], r2[i], 0x07060302u);
                *reinterpret_cast<uint2*>(base + v_lds[2 * i]) = lo;
                *reinterpret_cast<uint2*>(base + v_lds[2 * i + 1]) = hi;
            }
        }
    };

    // ---- per-lane LDS read offsets
    const int kf_off = l32 * T::K_RS + 16 * half * (D / 32);
    int vf_off[4];
    {
        const int x0 = (half ^ v_swz(l32)) & 7;
#pragma unroll
        for (int i = 0; i < 4; i++) vf_off[i] = T::K_BYTES + l32 * T::V_RS + (((2 * i) ^ x0) * 16);
    }

    // ---- running state: this lane's query row
    float m_i = -INFINITY;
    float l_i = half ? 0.0f : 1.0f;  // the two halves of a row sum to the reference's l = 1
    v16f o[T::DTILES];
#pragma unroll
    for (int dt = 0; dt < T::DTILES; dt++)
#pragma unroll
        for (int i = 0; i < 16; i++) o[dt][i] = 0.0f;

    // Mask entries of a step are fetched one step ahead, like the K/V tiles, wherever a run of four
    // keys can be read with one load (contiguous, aligned mask rows; runs that reach past kv_len are
    // read entry by entry when they are used).
    const int64_t mrow = MODE >= MODE_MASK_BOOL ? (int64_t)b * a.ms_b + (int64_t)h * a.ms_h + (int64_t)my_m * a.ms_m : 0;
    uint32_t mw_cur[8], mw_nxt[8];
    float4 mf_cur[8], mf_nxt[8];
    auto run_start = [&](int step, int r) { return step * BN + 32 * (r >> 2) + 8 * (r & 3) + 4 * half; };
    auto load_mask = [&](int step, uint32_t (&mw)[8], float4 (&mf)[8]) {
        if (MODE < MODE_MASK_BOOL || !a.mask_vec || !row_ok) return;
#pragma unroll
        for (int r = 0; r < 8; r++) {
            const int nb = run_start(step, r);
            if (nb + 3 < a.N) {
                if (MODE == MODE_MASK_BOOL) mw[r] = *reinterpret_cast<const uint32_t*>(static_cast<const uint8_t*>(a.mask) + mrow + nb);
                else mf[r] = mask_run4(a, mrow + nb);
            }
        }
    };

    if (nsteps > 0) {
        load_tile(0);
        load_mask(0, mw_cur, mf_cur);
        store_tile(0);
    }
    __syncthreads();

    for (int step = 0; step < nsteps; step++) {
        const int buf = step & 1;
        const bool more = step + 1 < nsteps;
        if (more) {
            load_tile(step + 1);
            load_mask(step + 1, mw_nxt, mf_nxt);
        }
        const unsigned char* base = smem + buf * T::STAGE;
        const int n0 = step * BN;

        // generic masks: fetch this lane's 32 mask entries, decide the tile skip (bool only)
        float madd[2][16];
        bool skip = false;
        if (MODE >= MODE_MASK_BOOL) {
            int any = 0;
            // one entry: visibility / additive value of key n for this lane's row (mv: the loaded mask entry)
            auto entry = [&](int kt, int i, int n, bool inb, bool mb, float mf, bool track) {
                bool keep = inb;
                if (a.causal) keep = keep && (n <= my_m + (a.N - a.M));
                if (MODE == MODE_MASK_BOOL) {
                    keep = keep && mb;
                    madd[kt][i] = keep ? 0.0f : kMasked;
                } else {
                    float add = inb ? mf : kMasked;
                    if (a.causal && inb && !keep) add += kMasked;
                    madd[kt][i] = add;
                }
                if (track) any |= keep;  // feeds the tile-skip vote (bool masks and causal only)
            };
#pragma unroll
            for (int kt = 0; kt < 2; kt++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    // the lane's keys come in runs of four consecutive ones
                    const int nb = n0 + 32 * kt + 8 * g + 4 * half;
                    if (a.mask_vec && row_ok && nb + 3 < a.N) {
                        if (MODE == MODE_MASK_BOOL) {
                            const uint32_t w = mw_cur[4 * kt + g];
                            if (!a.causal) any |= (w != 0u);
#pragma unroll
                            for (int e = 0; e < 4; e++) entry(kt, 4 * g + e, nb + e, true, ((w >> (8 * e)) & 0xffu) != 0, 0.0f, a.causal != 0);
                        } else {
                            const float4 w = mf_cur[4 * kt + g];
                            const float wf[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
                            for (int e = 0; e < 4; e++) entry(kt, 4 * g + e, nb + e, true, false, wf[e], a.causal != 0);
                        }
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            const int n = nb + e;
                            const bool inb = row_ok && n < a.N;
                            bool mb = false;
                            float mf = 0.0f;
                            if (inb) {
                                if (MODE == MODE_MASK_BOOL) mb = static_cast<const uint8_t*>(a.mask)[mrow + (int64_t)n * a.ms_n] != 0;
                                else mf = mask_entry(a, mrow + (int64_t)n * a.ms_n);
                            }
                            entry(kt, 4 * g + e, n, inb, mb, mf, true);
                        }
                    }
                }
            if (MODE == MODE_MASK_BOOL || a.causal) skip = !__syncthreads_or(any);
        }

        if (!skip) {
            // ---- S^T = K . Q^T
            v16i sacc[2];
#pragma unroll
            for (int kt = 0; kt < 2; kt++) {
#pragma unroll
                for (int i = 0; i < 16; i++) sacc[kt][i] = 0;
#pragma unroll
                for (int t = 0; t < T::KSTEPS; t++) {
                    const v4i kf = *reinterpret_cast<const v4i*>(base + kf_off + 32 * kt * T::K_RS + 16 * t);
                    sacc[kt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(kf, qf[t], sacc[kt], 0, 0, 0);
                }
            }

            // ---- online softmax (base 2), one row per lane
            const float sc = qs * ksp[step];
            float s[2][16];
            float rmax = -INFINITY;
            bool plain = (MODE == MODE_PLAIN) && (n0 + BN <= a.N);
            if (MODE == MODE_CAUSAL) plain = (n0 + BN <= a.N) && (n0 + BN - 1 <= m0 + 32 * wave + (a.N - a.M));
            if (plain) {
                // no element needs masking: fold the dequantization into the exponent's fma
#pragma unroll
                for (int kt = 0; kt < 2; kt++)
#pragma unroll
                    for (int i = 0; i < 16; i++) {
                        s[kt][i] = (float)sacc[kt][i];
                        rmax = fmaxf(rmax, s[kt][i]);
                    }
                rmax = xhalf_max(rmax) * sc;
            } else {
#pragma unroll
                for (int kt = 0; kt < 2; kt++)
#pragma unroll
                    for (int i = 0; i < 16; i++) {
                        float x;
                        if (MODE >= MODE_MASK_BOOL) {
                            x = __builtin_fmaf((float)sacc[kt][i], sc, madd[kt][i]);
                        } else {
                            x = (float)sacc[kt][i] * sc;
                            const int n = n0 + 32 * kt + 8 * (i >> 2) + 4 * half + (i & 3);
                            bool keep = n < a.N;
                            if (MODE == MODE_CAUSAL) keep = keep && (n <= my_m + (a.N - a.M));
                            x += keep ? 0.0f : kMasked;
                        }
                        s[kt][i] = x;
                        rmax = fmaxf(rmax, x);
                    }
                rmax = xhalf_max(rmax);
            }
            // The running maximum is only advanced (and O, l rescaled) when some row of this wave
            // moved by more than kTau; otherwise exponentials are taken against the stale maximum
            // (p <= 2^kTau, exact in the final o = O / l and lse = log2(l) + m).
            const float m_new = fmaxf(m_i, rmax);
            if (__builtin_amdgcn_ballot_w64(m_new - m_i > kTau) != 0) {
                const float alpha = __builtin_amdgcn_exp2f(m_i - m_new);
                l_i *= alpha;
                m_i = m_new;
#pragma unroll
                for (int dt = 0; dt < T::DTILES; dt++)
#pragma unroll
                    for (int i = 0; i < 16; i++) o[dt][i] *= alpha;
            }
            if (plain) {
#pragma unroll
                for (int kt = 0; kt < 2; kt++)
#pragma unroll
                    for (int i = 0; i < 16; i++) s[kt][i] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kt][i], sc, -m_i));
            } else {
#pragma unroll
                for (int kt = 0; kt < 2; kt++)
#pragma unroll
                    for (int i = 0; i < 16; i++) s[kt][i] = __builtin_amdgcn_exp2f(s[kt][i] - m_i);
            }

            // ---- P^T as the B operand: k-step t' of 16 keys takes S^T registers 8(t'&1) .. +7 of tile t'>>1.
            //      The row sum is taken over the rounded P (pairs through v_dot2), so that numerator and
            //      denominator of o = O / l see the same weights.
            vec16 pf[4];
            float lsum = 0.0f;
#pragma unroll
            for (int tp = 0; tp < 4; tp++) {
#pragma unroll
                for (int c = 0; c < 8; c++) pf[tp][c] = (VT)s[tp >> 1][8 * (tp & 1) + c];
#pragma unroll
                for (int c = 0; c < 4; c++) lsum = PVT::dot2_ones(pf[tp], c, lsum);
            }
            l_i += lsum;

            // ---- O^T += V^T . P^T
#pragma unroll
            for (int dt = 0; dt < T::DTILES; dt++)
#pragma unroll
                for (int tp = 0; tp < 4; tp++) {
                    const vec16 vf = *reinterpret_cast<const vec16*>(base + vf_off[tp ^ (2 * (dt & 1))] + dt * 32 * T::V_RS);
                    o[dt] = PVT::mfma(vf, pf[tp], o[dt]);
                }
        }

        if (more) store_tile(buf ^ 1);
        if (MODE == MODE_MASK_BOOL) {
#pragma unroll
            for (int r = 0; r < 8; r++) mw_cur[r] = mw_nxt[r];
        } else if (MODE == MODE_MASK_F32) {
#pragma unroll
            for (int r = 0; r < 8; r++) mf_cur[r] = mf_nxt[r];
        }
        __syncthreads();
    }

    // ---- epilogue: O = O^T / l, lse = log2(l) + m
    const float l_tot = xhalf_sum(l_i);
    const float inv = 1.0f / l_tot;
    if (row_ok) {
        const int64_t obase = (int64_t)b * a.os_b + (int64_t)h * a.os_h + (int64_t)my_m * a.os_n;
#pragma unroll
        for (int dt = 0; dt < T::DTILES; dt++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int d = 32 * dt + 8 * g + 4 * half;
                float r[4];
#pragma unroll
                for (int i = 0; i < 4; i++) r[i] = o[dt][4 * g + i] * inv;
                if (a.out_dt == SAGE_BF16) {
                    typedef __bf16 b4 __attribute__((ext_vector_type(4)));
                    b4 w = {(__bf16)r[0], (__bf16)r[1], (__bf16)r[2], (__bf16)r[3]};
                    *reinterpret_cast<b4*>(static_cast<__bf16*>(a.out) + obase + d) = w;
                } else if (a.out_dt == SAGE_F16) {
                    typedef _Float16 h4 __attribute__((ext_vector_type(4)));
                    h4 w = {(_Float16)r[0], (_Float16)r[1], (_Float16)r[2], (_Float16)r[3]};
                    *reinterpret_cast<h4*>(static_cast<_Float16*>(a.out) + obase + d) = w;
                } else {
                    *reinterpret_cast<v4f*>(static_cast<float*>(a.out) + obase + d) = v4f{r[0], r[1], r[2], r[3]};
                }
            }
        if (a.lse && half == 0) a.lse[((int64_t)b * a.Hq + h) * a.M + my_m] = __builtin_log2f(l_tot) + m_i;
    }
}

template <int D, typename VT>
int launch_mode(const AttnArgs& a, int mode, hipStream_t stream) {
    dim3 grid((unsigned)a.total_wg), block(kThreads);
    switch (mode) {
        case MODE_PLAIN: hipLaunchKernelGGL((sage_attn_fwd_kernel<D, VT, MODE_PLAIN>), grid, block, 0, stream, a); break;
        case MODE_CAUSAL: hipLaunchKernelGGL((sage_attn_fwd_kernel<D, VT, MODE_CAUSAL>), grid, block, 0, stream, a); break;
        case MODE_MASK_BOOL: hipLaunchKernelGGL((sage_attn_fwd_kernel<D, VT, MODE_MASK_BOOL>), grid, block, 0, stream, a); break;
        default: hipLaunchKernelGGL((sage_attn_fwd_kernel<D, VT, MODE_MASK_F32>), grid, block, 0, stream, a); break;
    }
    return check_launch("sage_attn_fwd_kernel");
}

}  // namespace

namespace {
// The calls the pipelined kernel serves without a mask tensor are the ones whose keys can be split.
int attn_key_splits(const sage_attn_params& p) {
    if (p.mask_kind != SAGE_MASK_NONE || (p.causal && p.qo_len > p.kv_len)) return 1;
    return attn::plan_key_split(p.batch, p.heads_q, p.qo_len, p.kv_len, p.causal != 0);
}
}  // namespace

int64_t attn_split_workspace_bytes(const sage_attn_params& p) {
    return attn::key_split_workspace_bytes(attn_key_splits(p), p.batch, p.heads_q, p.qo_len, p.head_dim);
}

int launch_attn(const sage_attn_params& p, void* workspace, int64_t workspace_bytes, hipStream_t stream) {
    AttnArgs a{};
    a.q = (const int8_t*)p.q.ptr; a.k = (const int8_t*)p.k.ptr; a.v = p.v.ptr; a.out = p.out.ptr;
    a.q_scale = p.q_scale; a.k_scale = p.k_scale; a.lse = p.lse; a.mask = p.mask;
    a.qs_b = p.q.stride_b; a.qs_h = p.q.stride_h; a.qs_n = p.q.stride_n;
    a.ks_b = p.k.stride_b; a.ks_h = p.k.stride_h; a.ks_n = p.k.stride_n;
    a.vs_b = p.v.stride_b; a.vs_h = p.v.stride_h; a.vs_n = p.v.stride_n;
    a.os_b = p.out.stride_b; a.os_h = p.out.stride_h; a.os_n = p.out.stride_n;
    a.ms_b = p.mask_stride_b; a.ms_h = p.mask_stride_h; a.ms_m = p.mask_stride_m; a.ms_n = p.mask_stride_n;
    a.Hq = (int)p.heads_q; a.Hkv = (int)p.heads_kv; a.M = (int)p.qo_len; a.N = (int)p.kv_len;
    a.nq = (int)((p.qo_len + BM - 1) / BM); a.nk = (int)((p.kv_len + BN - 1) / BN);
    a.groups = (int)(p.heads_q / p.heads_kv);
    a.out_dt = p.out_dtype; a.causal = p.causal ? 1 : 0;
    a.lse_mul = 1.0f;
    const bool is_bool = p.mask_kind == SAGE_MASK_BOOL || p.mask_kind == SAGE_MASK_BOOL_PADDED ||
                         p.mask_kind == SAGE_MASK_BOOL_PADDED_CAUSAL;
    a.mask_padded = p.mask_kind == SAGE_MASK_BOOL_PADDED || p.mask_kind == SAGE_MASK_BOOL_PADDED_CAUSAL ||
                    p.mask_kind == SAGE_MASK_F16_PADDED || p.mask_kind == SAGE_MASK_BF16_PADDED ||
                    p.mask_kind == SAGE_MASK_F32_PADDED;
    a.mask_causal = p.mask_kind == SAGE_MASK_BOOL_PADDED_CAUSAL;
    const bool f16 = p.mask_kind == SAGE_MASK_F16 || p.mask_kind == SAGE_MASK_F16_PADDED;
    const bool bf16 = p.mask_kind == SAGE_MASK_BF16 || p.mask_kind == SAGE_MASK_BF16_PADDED;
    const bool additive = p.mask_kind == SAGE_MASK_F32 || p.mask_kind == SAGE_MASK_F32_PADDED || f16 || bf16;
    a.mask_dt = f16 ? SAGE_F16 : bf16 ? SAGE_BF16 : SAGE_F32;
    if (p.mask_kind != SAGE_MASK_NONE && p.mask_stride_n == 1) {
        // runs of four entries are read with one load where they are naturally aligned
        const int64_t esz = is_bool ? 1 : dtype_bytes(a.mask_dt), align = 4 * esz;
        a.mask_vec = ((uintptr_t)p.mask % align) == 0 && (p.mask_stride_b * esz) % align == 0 &&
                     (p.mask_stride_h * esz) % align == 0 && (p.mask_stride_m * esz) % align == 0;
    }
    const int64_t total = p.batch * p.heads_q * a.nq;
    if (total > 0x7fffffffLL || p.qo_len > 0x7fffffffLL - BM || p.kv_len > 0x7fffffffLL - BN)
        return fail(SAGE_E_UNSUPPORTED, "sage_attn_fwd: problem too large for 32-bit tile indices");
    if (p.k.stride_n < 0 || p.v.stride_n < 0 || (int64_t)BN * p.k.stride_n >= (1LL << 30) ||
        (int64_t)BN * p.v.stride_n >= (1LL << 29))
        return fail(SAGE_E_UNSUPPORTED, "sage_attn_fwd: k/v sequence stride out of range for 32-bit tile offsets");
    a.total_wg = (int)total;
    a.nsplit = 1; a.split_steps = a.nk;
    a.head_tile = 1;
    if (p.mask_kind != SAGE_MASK_NONE && p.mask_stride_h == 0 && p.heads_q > 1)
        a.head_tile = p.heads_q % 8 == 0 ? 8 : p.heads_q % 4 == 0 ? 4 : p.heads_q % 2 == 0 ? 2 : 1;
    int mode = MODE_PLAIN;
    if (is_bool) mode = MODE_MASK_BOOL;
    else if (additive) mode = MODE_MASK_F32;
    else if (p.causal) mode = MODE_CAUSAL;
    const bool fast = p.mask_kind == SAGE_MASK_NONE && (!p.causal || p.qo_len <= p.kv_len);
    if (fast) {
        const int nsplit = workspace ? attn_key_splits(p) : 1;
        if (nsplit > 1 && workspace_bytes >= attn::key_split_workspace_bytes(nsplit, p.batch, p.heads_q, p.qo_len, p.head_dim)) {
            if (total * nsplit > 0x7fffffffLL) return fail(SAGE_E_UNSUPPORTED, "sage_attn_fwd: problem too large for 32-bit tile indices");
            AttnArgs s = a;
            attn::apply_key_split(s, nsplit, p.batch, (int)p.head_dim, workspace);
            if (int rc = attn::launch_fast(s, (int)p.head_dim, p.v_dtype, p.causal != 0, stream)) return rc;
            return attn::launch_split_combine(s, a, (int)p.head_dim, p.batch, stream);
        }
        return attn::launch_fast(a, (int)p.head_dim, p.v_dtype, p.causal != 0, stream);
    }
    a.mask_additive = additive;
    if ((is_bool && attn::fast_serves_mask(a, 1)) || (additive && attn::fast_serves_mask(a, dtype_bytes(a.mask_dt))))
        return attn::launch_fast_masked(a, (int)p.head_dim, p.v_dtype, stream);
    if (p.head_dim == 128) {
        return p.v_dtype == SAGE_BF16 ? launch_mode<128, __bf16>(a, mode, stream)
                                      : launch_mode<128, _Float16>(a, mode, stream);
    }
    return p.v_dtype == SAGE_BF16 ? launch_mode<64, __bf16>(a, mode, stream)
                                  : launch_mode<64, _Float16>(a, mode, stream);
}

}  // namespace sage
