// Software-pipelined SageAttention forward for gfx950: the common case (no mask tensor, kv_len a
// multiple of 64, causal only with qo_len <= kv_len).  Same arithmetic contract as the general
// kernel in attn_fwd.hip (FlagAttention src/flag_attn/sage_attention/attn_qk_int8_per_block.py:
// 20-127); what differs is how the work is laid out in time.
//
// Per workgroup: 8 waves x 32 query rows (two q_scale blocks, so that every K/V tile staged in LDS
// serves 256 rows); per step: 64 keys.  Every wave computes the transposed
// products S^T = K.Q^T (8 x v_mfma_i32_32x32x32_i8) and O^T += V^T.P^T (16 x v_mfma_f32_32x32x16)
// so that a lane owns one query row and P never leaves registers.
//
// * V is staged in LDS as it lies in memory ([key][channel], rows padded by 64 bytes) and read
//   with ds_read_b64_tr_b16, which hands each lane four consecutive keys of one channel: exactly
//   the A operand of the P.V MFMA, with no shuffling instructions.
// * Every wave alternates between a VALU phase (exponentials of step j) and an MFMA phase (Q.K^T of
//   step j+1 and P.V of step j back to back, with the row sums of P and the raw row maximum of
//   step j+1 riding in the shadow of the matrix instructions).  The two waves that share a SIMD
//   run half a step apart, so the matrix core and the VALU are both kept busy; phases are
//   separated by workgroup barriers (two per step).
// * K of step j+3 and V of step j+2 are fetched from global memory into registers during the MFMA
//   phase of step j, one 16-byte piece per slot, right after the piece fetched a step earlier has
//   been handed to LDS; nothing is waited for at the end of a step.
// * The int32 Q.K^T accumulators start from the bit pattern of 1.5 * 2^23, so their bits ARE the
//   float kBias + dot and no int -> float conversion is issued; the two score register sets swap
//   roles every step (the loop body exists for both parities).
// * The running maximum is advanced lazily (kTau) so the O accumulators are rescaled only on the
//   rare steps where a row maximum jumps.
#include <utility>

#include "attn_common.h"

namespace sage {
namespace attn {
namespace {

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) s16x4* lds_s16x4_ptr;
typedef unsigned v2u __attribute__((ext_vector_type(2)));

// compile-time loops: f(IC<0>{}), f(IC<1>{}), ...
template <int I> struct IC { static constexpr int value = I; };
template <typename Fn, int... Is>
__device__ __forceinline__ void sfor_impl(Fn&& f, std::integer_sequence<int, Is...>) { (f(IC<Is>{}), ...); }
template <int N, typename Fn>
__device__ __forceinline__ void sfor(Fn&& f) { sfor_impl(f, std::make_integer_sequence<int, N>{}); }

constexpr int kBiasBits = 0x4B400000;  // 12582912.0f = 1.5 * 2^23
constexpr float kBias = 12582912.0f;
// exp2(fma(kBias + dot, sc, -(kBias * sc + m))) loses ulp(kBias * sc) / 2 in the exponent; above this
// product the bias is subtracted explicitly instead.
constexpr float kBiasFoldLimit = 8192.0f;
#ifndef SAGE_WAVES
#define SAGE_WAVES 8
#endif
constexpr int kFastWaves = SAGE_WAVES;            // waves per workgroup, 32 query rows each
constexpr int kFastThreads = 64 * kFastWaves;
constexpr int kFastRows = 32 * kFastWaves;        // query rows per workgroup
constexpr int kFastWgPerCu = 8 / kFastWaves;      // two waves per SIMD either way

template <int D>
struct FT {
    static constexpr int KSTEPS = D / 32;
    static constexpr int DTILES = D / 32;
    static constexpr int K_RS = D + 16;       // bytes per K row in LDS
    static constexpr int K_BYTES = BN * K_RS;
    static constexpr int V_RS = 2 * D + 64;   // bytes per V row in LDS
    static constexpr int V_BYTES = BN * V_RS;
    static constexpr int K_ITEMS = BN * (D / 16);  // 16-byte pieces per K tile
    static constexpr int K_LOADS = (K_ITEMS + kFastThreads - 1) / kFastThreads;
    static constexpr int V_LOADS = BN * (D / 8) / kFastThreads;
    static constexpr int V_BASE = 2 * K_BYTES;
    static constexpr int TOTAL = 2 * K_BYTES + 2 * V_BYTES;
};

template <typename VT>
__device__ __forceinline__ typename PV<VT>::vec tr_pair(const unsigned char* p0, const unsigned char* p1) {
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)p0);
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)p1);
    const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(typename PV<VT>::vec, both);
}

template <int D, typename VT, bool CAUSAL>
__global__ __launch_bounds__(kFastThreads, kFastWgPerCu) void sage_attn_fwd_fast_kernel(AttnArgs a, int nq2) {
    using F = FT<D>;
    using PVT = PV<VT>;
    using vec16 = typename PVT::vec;
    __shared__ __attribute__((aligned(16))) unsigned char smem[F::TOTAL];

    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int l32 = lane & 31;
    const int half = lane >> 5;

    // workgroup -> (batch, head, q-block); consecutive logical ids stay on one XCD (8 XCDs, round robin)
    int wg = blockIdx.x;
    if ((a.total_wg & 7) == 0) wg = (wg & 7) * (a.total_wg >> 3) + (wg >> 3);
    int iq = wg % nq2;
    if (CAUSAL) iq = nq2 - 1 - iq;  // longest rows first
    const int h = (wg / nq2) % a.Hq;
    const int b = wg / (nq2 * a.Hq);
    const int hk = h / a.groups;
    const int m0 = iq * kFastRows;
    const int my_m = m0 + 32 * wave + l32;
    const bool row_ok = my_m < a.M;
    const int shift = a.N - a.M;  // causal: key n is visible to row m iff n <= m + shift

    int nsteps = a.nk;
    if (CAUSAL) {
        const int last_row = min(m0 + kFastRows, a.M) - 1;
        nsteps = min(nsteps, (last_row + shift + BN) / BN);  // >= 1 because qo_len <= kv_len
    }

    // Q fragments: lane (row l32, half) holds channels half*D/2 + 16t .. +15 of k-step t
    v4i qf[F::KSTEPS];
    {
        const int8_t* qp = a.q + (int64_t)b * a.qs_b + (int64_t)h * a.qs_h + (int64_t)my_m * a.qs_n + half * (D / 2);
#pragma unroll
        for (int t = 0; t < F::KSTEPS; t++)
            qf[t] = row_ok ? *reinterpret_cast<const v4i*>(qp + 16 * t) : v4i{0, 0, 0, 0};
    }
    const float qs = a.q_scale[((int64_t)b * a.Hq + h) * a.nq + min((kFastRows / BM) * iq + (wave >> 2), a.nq - 1)];
    const float* ksp = a.k_scale + ((int64_t)b * a.Hkv + hk) * a.nk;
    const int8_t* kg = a.k + (int64_t)b * a.ks_b + (int64_t)hk * a.ks_h;
    const VT* vg = static_cast<const VT*>(a.v) + (int64_t)b * a.vs_b + (int64_t)hk * a.vs_h;

    // staging: 16-byte pieces, consecutive lanes along a row
    int k_goff[F::K_LOADS], k_lds[F::K_LOADS], v_goff[F::V_LOADS], v_lds[F::V_LOADS];
    const bool k_worker = tid < F::K_ITEMS;
#pragma unroll
    for (int j = 0; j < F::K_LOADS; j++) {
        const int id = (tid + kFastThreads * j) % F::K_ITEMS;
        const int row = id / (D / 16), c = id % (D / 16);
        k_goff[j] = row * (int)a.ks_n + 16 * c;
        k_lds[j] = row * F::K_RS + 16 * c;
    }
#pragma unroll
    for (int i = 0; i < F::V_LOADS; i++) {
        const int id = tid + kFastThreads * i;
        const int row = id / (D / 8), c = id % (D / 8);
        v_goff[i] = row * (int)a.vs_n + 8 * c;
        v_lds[i] = F::V_BASE + row * F::V_RS + 16 * c;
    }
    v4i kreg[F::K_LOADS];
    v4i vreg[F::V_LOADS];  // native vectors: a struct type here ends up as a stack array in LDS
    auto load_k = [&](int tile) {
        const int8_t* kt = kg + (int64_t)tile * BN * a.ks_n;
        if (F::K_ITEMS >= kFastThreads || k_worker) {
#pragma unroll
            for (int j = 0; j < F::K_LOADS; j++) kreg[j] = *reinterpret_cast<const v4i*>(kt + k_goff[j]);
        }
    };
    auto load_v = [&](int tile) {
        const VT* vt = vg + (int64_t)tile * BN * a.vs_n;
#pragma unroll
        for (int i = 0; i < F::V_LOADS; i++) vreg[i] = *reinterpret_cast<const v4i*>(vt + v_goff[i]);
    };
    auto store_k = [&](int buf) {
        if (F::K_ITEMS >= kFastThreads || k_worker) {
#pragma unroll
            for (int j = 0; j < F::K_LOADS; j++) *reinterpret_cast<v4i*>(smem + buf * F::K_BYTES + k_lds[j]) = kreg[j];
        }
    };
    // piecewise variants used inside the step pipeline (one 16-byte piece per call)
    // (uniform 64-bit tile pointer + unsigned 32-bit lane offset: one scalar-base load instruction)
    auto restage_k = [&](auto jc, int buf, const unsigned char* tile) {
        constexpr int j = decltype(jc)::value;
        if (F::K_ITEMS >= kFastThreads || k_worker) {
            *reinterpret_cast<v4i*>(smem + buf * F::K_BYTES + k_lds[j]) = kreg[j];
            kreg[j] = *reinterpret_cast<const v4i*>(tile + (unsigned)k_goff[j]);
        }
    };
    auto restage_v = [&](auto ic, int buf, const unsigned char* tile) {
        constexpr int i = decltype(ic)::value;
        *reinterpret_cast<v4i*>(smem + buf * F::V_BYTES + v_lds[i]) = vreg[i];
        vreg[i] = *reinterpret_cast<const v4i*>(tile + 2u * (unsigned)v_goff[i]);
    };
    auto store_v = [&](int buf) {
#pragma unroll
        for (int i = 0; i < F::V_LOADS; i++) *reinterpret_cast<v4i*>(smem + buf * F::V_BYTES + v_lds[i]) = vreg[i];
    };

    // fragment read offsets
    const int kf_off = l32 * F::K_RS + 16 * half * (D / 32);
    // ds_read_b64_tr_b16: in each group of 16 lanes, lane 4s+a supplies keys row s, channels 4a..4a+3,
    // and lane i receives channel i of the four rows.  Groups: (channels 0-15 | 16-31) x (half 0 | 1).
    const int vtr_off = F::V_BASE + (4 * half + ((lane >> 2) & 3)) * F::V_RS + (16 * ((lane >> 4) & 1) + 4 * (lane & 3)) * 2;

    // The int32 accumulators start from the bit pattern of the float 1.5 * 2^23: since |dot| < 2^22,
    // accumulator bits reinterpreted as fp32 ARE kBias + dot, so no int -> float conversion is needed.
    v16i bias16;
#pragma unroll
    for (int i = 0; i < 16; i++) {
        int b;  // materialised once through an opaque move, so the block stays in VGPRs for the whole kernel
        asm volatile("v_mov_b32 %0, %1" : "=v"(b) : "s"(kBiasBits));
        bias16[i] = b;
    }
    auto qk_tile = [&](const unsigned char* kbase, int kt) {
        v16i acc = bias16;
#pragma unroll
        for (int t = 0; t < F::KSTEPS; t++) {
            const v4i kf = *reinterpret_cast<const v4i*>(kbase + kf_off + 32 * kt * F::K_RS + 16 * t);
            acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(kf, qf[t], acc, 0, 0, 0);
        }
        return acc;
    };

    float m_i = -INFINITY;
    float l_i = half ? 0.0f : 1.0f;  // the two halves of a row sum to the reference's initial l = 1
    v16f o[F::DTILES];
#pragma unroll
    for (int dt = 0; dt < F::DTILES; dt++)
#pragma unroll
        for (int i = 0; i < 16; i++) o[dt][i] = 0.0f;

    // ---- the step pipeline -----------------------------------------------------------------
    // The MFMA phase of a step issues QK_SLOTS + PV_SLOTS matrix instructions.  Each "slot" is one
    // MFMA plus the few VALU / LDS instructions that run in its shadow, fenced so that the order
    // written here is the order issued; LDS fragment reads are issued a few slots ahead of the
    // MFMA that consumes them.
    constexpr int QK_SLOTS = 2 * F::KSTEPS;
    constexpr int PV_SLOTS = 4 * F::DTILES;
    constexpr int NSLOTS = QK_SLOTS + PV_SLOTS;
#ifndef SAGE_KDIST
#define SAGE_KDIST 4
#endif
#ifndef SAGE_VDIST
#define SAGE_VDIST 3
#endif
    constexpr int KDIST = SAGE_KDIST < QK_SLOTS ? SAGE_KDIST : QK_SLOTS;      // K fragments in flight
    constexpr int VDIST = SAGE_VDIST < QK_SLOTS ? SAGE_VDIST : QK_SLOTS - 1;  // V fragments in flight
    static_assert(KDIST <= QK_SLOTS && VDIST < QK_SLOTS && 16 % QK_SLOTS == 0, "slot plan");

    // Scores live in two register sets that swap roles every step (the loop body is instantiated
    // for both parities), so the accumulators Q.K^T writes in one iteration are read in place by
    // the exponentials of the next one.
    v16i sbuf[2][2];  // [parity][32-key tile]: int32 accumulators whose bits are the float kBias + dot
    float raw_max;    // maximum of the current step's 32 biased scores of this lane
    float sc;         // q_scale * k_scale of the current step

    auto as_f = [](int bits) { return __builtin_bit_cast(float, bits); };
    auto head_unit = [&](auto pc, auto uc, int n0_next, bool masked, float& acc) {
        constexpr int P = decltype(pc)::value, u = decltype(uc)::value;
        constexpr int kt = u >> 2, i0 = 4 * (u & 3);
        float x[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int bits = sbuf[P][kt][i0 + e];  // (scalar copy: bit_cast of a vector element lvalue reads element 0)
            x[e] = as_f(bits);
            if (CAUSAL && masked) {
                const int i = i0 + e;
                const int n = n0_next + 32 * kt + 8 * (i >> 2) + 4 * half + (i & 3);
                x[e] = (n > my_m + shift) ? -INFINITY : x[e];
                sbuf[P][kt][i] = __builtin_bit_cast(int, x[e]);
            }
        }
        acc = fmaxf(fmaxf(acc, x[0]), x[1]);
        acc = fmaxf(fmaxf(acc, x[2]), x[3]);
        asm volatile("" ::"v"(acc));  // pin to this slot (otherwise sunk below the matrix instructions)
    };

    // ---- prologue: K0, V0, K1 in LDS; scores of step 0 in registers
    load_k(0);
    load_v(0);
    store_k(0);
    store_v(0);
    load_k(min(1, nsteps - 1));
    store_k(1);
    __syncthreads();
    load_k(min(2, nsteps - 1));  // stored to LDS at the top of the first iteration
    load_v(min(1, nsteps - 1));
    sbuf[0][0] = qk_tile(smem, 0);
    sbuf[0][1] = qk_tile(smem, 1);
    raw_max = -INFINITY;
    {
        const bool masked0 = CAUSAL && (BN - 1 > m0 + 32 * wave + shift);
        sfor<8>([&](auto uc) { head_unit(IC<0>{}, uc, 0, masked0, raw_max); });
    }
    sc = qs * ksp[0];
    if (CAUSAL) sc = fmaxf(sc, 1.17549435e-38f);  // keeps -inf * sc = -inf for hidden keys of an all-zero K block

#ifdef SAGE_PROF
    long long prof[4] = {0, 0, 0, 0};
#define PROF_T(v) const long long v = __builtin_readcyclecounter(); asm volatile("" ::: "memory")
#else
#define PROF_T(v)
#endif

    // tiles fetched during step 0 (K of step 3, V of step 2, clamped to the last step)
    const int64_t k_tile_bytes = (int64_t)BN * a.ks_n, v_tile_bytes = (int64_t)BN * a.vs_n * 2;
    const unsigned char* k_fetch = reinterpret_cast<const unsigned char*>(kg) + min(3, nsteps - 1) * k_tile_bytes;
    const unsigned char* v_fetch = reinterpret_cast<const unsigned char*>(vg) + min(2, nsteps - 1) * v_tile_bytes;

    // ---- one step.  Each wave alternates a VALU phase (exponentials of its step) and an MFMA phase
    // (Q.K^T of the next step, P.V of this one, with the row sums and the next step's raw maximum
    // in the shadow of the matrix instructions); the two waves that share a SIMD run half a step
    // apart (see the barrier before the loop), so one feeds the matrix core while the other
    // occupies the VALU.  Two barriers per step.
    auto body = [&](auto pc, int step) {
        constexpr int P = decltype(pc)::value;  // == step & 1
        const unsigned char* kb_next = smem + (1 - P) * F::K_BYTES + kf_off;
        const unsigned char* vb_cur = smem + P * F::V_BYTES + vtr_off;
        const int n0 = step * BN;
        PROF_T(t_top);
        (void)n0;

        // ===== VALU phase: exponentials of this step (scores in sbuf[P]; their raw maximum was
        //       taken in the shadow of the previous MFMA phase) =====
        const float rmx = raw_max;
        {
            const v2u sw = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(unsigned, rmx),
                                                            __builtin_bit_cast(unsigned, rmx), false, false);
            const float rmax = (fmaxf(__builtin_bit_cast(float, sw[0]), __builtin_bit_cast(float, sw[1])) - kBias) * sc;
            const float m_new = fmaxf(m_i, rmax);
            if (__builtin_amdgcn_ballot_w64(m_new - m_i > kTau) != 0) {
                const float alpha = __builtin_amdgcn_exp2f(m_i - m_new);
                l_i *= alpha;
                m_i = m_new;
#pragma unroll
                for (int dt = 0; dt < F::DTILES; dt++)
#pragma unroll
                    for (int i = 0; i < 16; i++) o[dt][i] *= alpha;
            }
        }
        float neg_m;
        if (kBias * sc < kBiasFoldLimit) {
            neg_m = __builtin_fmaf(-kBias, sc, -m_i);
        } else {
#pragma unroll
            for (int kt = 0; kt < 2; kt++)
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const int bits = sbuf[P][kt][i];
                    sbuf[P][kt][i] = __builtin_bit_cast(int, as_f(bits) - kBias);
                }
            neg_m = -m_i;
        }
        vec16 pf[4];
        float lsum = 0.0f;
        sfor<16>([&](auto uc) {
            constexpr int u = decltype(uc)::value;
            constexpr int tp = u >> 2, w = u & 3, kt = tp >> 1, i0 = 8 * (tp & 1) + 2 * w;
            const int b0 = sbuf[P][kt][i0], b1 = sbuf[P][kt][i0 + 1];
            const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(as_f(b0), sc, neg_m));
            const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(as_f(b1), sc, neg_m));
            pf[tp][2 * w] = (VT)p0;
            pf[tp][2 * w + 1] = (VT)p1;
#ifdef SAGE_DOT2_IN_VALU_PHASE
            lsum = PVT::dot2_ones(pf[tp], w, lsum);
#endif
        });
        sc = qs * ksp[min(step + 1, nsteps - 1)];
        if (CAUSAL) sc = fmaxf(sc, 1.17549435e-38f);
        __builtin_amdgcn_sched_barrier(0);
        PROF_T(t_head);
        __syncthreads();  // phase switch: this wave takes the matrix core
        PROF_T(t_slots);

        // ===== MFMA phase =====
#ifndef SAGE_NOPRIO
        __builtin_amdgcn_s_setprio(1);
#endif
        float raw_max_n = -INFINITY;
        const bool masked_n = CAUSAL && (n0 + 2 * BN - 1 > m0 + 32 * wave + shift);
        v4i kfr[QK_SLOTS];
        vec16 vfr[PV_SLOTS];
        auto read_k = [&](auto ic) {
            constexpr int i = decltype(ic)::value;
            kfr[i] = *reinterpret_cast<const v4i*>(kb_next + 32 * (i % 2) * F::K_RS + 16 * (i / 2));
        };
        auto read_v = [&](auto jc) {
            constexpr int j = decltype(jc)::value;
            const unsigned char* p0 = vb_cur + 16 * (j / F::DTILES) * F::V_RS + 64 * (j % F::DTILES);
            vfr[j] = tr_pair<VT>(p0, p0 + 8 * F::V_RS);
        };
        sfor<KDIST>(read_k);
        sfor<NSLOTS>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            if constexpr (i < QK_SLOTS) {
                constexpr int kt = i % 2, t = i / 2;  // alternate the two accumulation chains
                if constexpr (t == 0) {
                    sbuf[1 - P][kt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(kfr[i], qf[t], bias16, 0, 0, 0);
                } else {
                    sbuf[1 - P][kt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(kfr[i], qf[t], sbuf[1 - P][kt], 0, 0, 0);
                }
                if constexpr (i + KDIST < QK_SLOTS) read_k(IC<i + KDIST>{});
                if constexpr (i >= QK_SLOTS - VDIST) read_v(IC<i - (QK_SLOTS - VDIST)>{});
                // row sums of P ride in the shadow of the Q.K^T instructions
#ifndef SAGE_DOT2_IN_VALU_PHASE
                sfor<16 / QK_SLOTS>([&](auto rc) {
                    constexpr int u = i * (16 / QK_SLOTS) + decltype(rc)::value;
                    lsum = PVT::dot2_ones(pf[u >> 2], u & 3, lsum);
                    asm volatile("" ::"v"(lsum));
                });
#endif
            } else {
                constexpr int j = i - QK_SLOTS, tp = j / F::DTILES, dt = j % F::DTILES;
                o[dt] = PVT::mfma(vfr[j], pf[tp], o[dt]);
                if constexpr (j + VDIST < PV_SLOTS) read_v(IC<j + VDIST>{});
                if constexpr (j < F::K_LOADS) restage_k(IC<j>{}, P, k_fetch);
                else if constexpr (j < F::K_LOADS + F::V_LOADS) restage_v(IC<j - F::K_LOADS>{}, 1 - P, v_fetch);
                // raw maximum of the next step's scores (Q.K^T finished above) under the P.V instructions
                sfor<8 / PV_SLOTS + (8 % PV_SLOTS != 0)>([&](auto rc) {
                    constexpr int u = j * (8 / PV_SLOTS + (8 % PV_SLOTS != 0)) + decltype(rc)::value;
                    if constexpr (u < 8) {
                        if (CAUSAL && masked_n) head_unit(IC<1 - P>{}, IC<u>{}, n0 + BN, true, raw_max_n);
                        else head_unit(IC<1 - P>{}, IC<u>{}, n0 + BN, false, raw_max_n);
                    }
                });
            }
            __builtin_amdgcn_sched_barrier(0);
        });
        l_i += lsum;
        raw_max = raw_max_n;
        if (step + 4 < nsteps) k_fetch += k_tile_bytes;  // next iteration fetches K of step+4, V of step+3
        if (step + 3 < nsteps) v_fetch += v_tile_bytes;
#ifndef SAGE_NOPRIO
        __builtin_amdgcn_s_setprio(0);
#endif
        PROF_T(t_store);
        __syncthreads();  // phase switch: this wave goes back to the VALU
#ifdef SAGE_PROF
        {
            PROF_T(t_end);
            prof[0] += t_head - t_top; prof[1] += t_slots - t_head; prof[2] += t_store - t_slots; prof[3] += t_end - t_store;
        }
#endif
    };

    if (wave >= kFastWaves / 2) __syncthreads();  // second half of the waves runs one phase behind
    for (int step = 0; step < nsteps; step += 2) {
        body(IC<0>{}, step);
        if (step + 1 >= nsteps) break;
        body(IC<1>{}, step + 1);
    }
    if (wave < kFastWaves / 2) __syncthreads();

    // ---- epilogue: O = O^T / l, lse = log2(l) + m
    const float l_o = __shfl_xor(l_i, 32);
    const float l_tot = half ? (l_o + l_i) : (l_i + l_o);
    const float inv = 1.0f / l_tot;
    if (row_ok) {
        const int64_t obase = (int64_t)b * a.os_b + (int64_t)h * a.os_h + (int64_t)my_m * a.os_n;
#pragma unroll
        for (int dt = 0; dt < F::DTILES; dt++)
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
#ifndef SAGE_PROF
        if (a.lse && half == 0) a.lse[((int64_t)b * a.Hq + h) * a.M + my_m] = __builtin_log2f(l_tot) + m_i;
#endif
    }
#ifdef SAGE_PROF
    if (a.lse && lane == 0) {  // debug build: per-wave cycle totals of the loop phases replace the lse output
        float* dst = a.lse + ((int64_t)blockIdx.x * kFastWaves + wave) * 4;
        for (int i = 0; i < 4; i++) dst[i] = (float)prof[i];
    }
#endif
}

template <int D, typename VT>
int launch_causal(const AttnArgs& a, bool causal, hipStream_t stream) {
    AttnArgs b = a;
    const int nq2 = (a.M + kFastRows - 1) / kFastRows;
    b.total_wg = (int)((int64_t)a.total_wg / a.nq * nq2);
    dim3 grid((unsigned)b.total_wg), block(kFastThreads);
    if (causal) hipLaunchKernelGGL((sage_attn_fwd_fast_kernel<D, VT, true>), grid, block, 0, stream, b, nq2);
    else hipLaunchKernelGGL((sage_attn_fwd_fast_kernel<D, VT, false>), grid, block, 0, stream, b, nq2);
    return check_launch("sage_attn_fwd_fast_kernel");
}

}  // namespace

int launch_fast(const AttnArgs& a, int head_dim, int v_dtype, bool causal, hipStream_t stream) {
    if (head_dim == 128)
        return v_dtype == SAGE_BF16 ? launch_causal<128, __bf16>(a, causal, stream)
                                    : launch_causal<128, _Float16>(a, causal, stream);
    return v_dtype == SAGE_BF16 ? launch_causal<64, __bf16>(a, causal, stream)
                                : launch_causal<64, _Float16>(a, causal, stream);
}

}  // namespace attn
}  // namespace sage
