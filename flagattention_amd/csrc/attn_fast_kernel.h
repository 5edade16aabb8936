// The software-pipelined attention forward kernel of libsage_attention_hip.so (gfx950), as a template
// over head_dim, the 16-bit type of V and P, whether keys can be hidden, and the width of Q and K
// elements.  Included by the two translation units that instantiate it: attn_fwd_fast.hip (int8 Q, K:
// SageAttention) and flash_fwd.hip (16-bit Q, K: dense attention).
//
// Per workgroup: 8 waves x 32 query rows (two q_scale blocks of the int8 path, so that every K/V tile
// staged in LDS serves 256 rows); per step: 64 keys (one k_scale block).  Every wave computes the transposed
// products S^T = K.Q^T (8 x v_mfma_i32_32x32x32_i8, or 16 x v_mfma_f32_32x32x16 for 16-bit Q and K, at
// head_dim 128) and O^T += V^T.P^T (16 x v_mfma_f32_32x32x16)
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
// * (int8) The int32 Q.K^T accumulators start from the bit pattern of 1.5 * 2^23, so their bits ARE the
//   float kBias + dot and no int -> float conversion is issued; the two score register sets swap
//   roles every step (the loop body exists for both parities).
// * No row maximum is taken per step: exponentials use the reference point the row already has
//   (the maximum of its first tile to begin with), and a step whose row sums come out large is
//   redone against its true maximum before any P.V instruction of it has been issued.  The row
//   sums are needed anyway, so the common step pays nothing for the check but a compare.
// * 16-bit outputs are transposed through LDS and written as whole rows.
// * Under the causal flag a workgroup takes two q-blocks of its head (the longest remaining and the
//   shortest), so that all workgroups of a launch run the same number of steps.
#pragma once
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
// A lane's 32 P of one step sum to less than this, or the step is redone.  fp16 P: no P may pass 65504.  bf16 P has
// the exponent range of fp32: the limit only keeps 2^60 * |V| * kv_len and the row sums far inside that range, so a
// row maximum may run up to 60 log2 units ahead of the row's reference point before a step has to be redone.
template <typename VT> constexpr float sum_limit() { return 32768.0f; }
template <> constexpr float sum_limit<__bf16>() { return 0x1p60f; }
constexpr int kFastWaves = 8;                     // waves per workgroup, 32 query rows each
constexpr int kFastThreads = 64 * kFastWaves;
static_assert(kFastRows == 32 * kFastWaves, "query rows per workgroup");
constexpr int kFastWgPerCu = 8 / kFastWaves;      // two waves per SIMD either way

// LDS tiles are unpadded ([64 keys][row bytes]) because they are filled by direct-to-LDS loads, which
// write 1 KB per wave instruction contiguously; bank conflicts are avoided by XOR-swizzling the
// 16-byte chunk index of every row (the swizzle is applied on the global-address side of the load
// and undone by the fragment reads).
template <int D, int QB>
struct FT {
    static constexpr int K_RS = D * QB;       // bytes per K row in LDS (QB bytes per element: int8 or 16-bit)
    static constexpr int KSTEPS = K_RS / 32;  // Q.K^T matrix instructions per 32-key tile: 32 bytes of a row each
    static constexpr int DTILES = D / 32;
    static constexpr int K_BYTES = BN * K_RS;
    static constexpr int V_RS = 2 * D;        // bytes per V row in LDS (16-bit)
    static constexpr int V_BYTES = BN * V_RS;
    static constexpr int KCPR = K_RS / 16;    // 16-byte chunks per K row
    static constexpr int VCPR = V_RS / 16;
    static constexpr int K_INSTR = K_BYTES / 1024;  // wave-level 1 KB loads per K tile (8 | 4)
    static constexpr int V_INSTR = V_BYTES / 1024;  // (16 | 8)
    static constexpr int NBUF = 4;            // tiles of K (and of V) resident in LDS
    static constexpr int V_BASE = NBUF * K_BYTES;
    static constexpr int TOTAL = NBUF * (K_BYTES + V_BYTES);
    static constexpr int NK = K_INSTR >= kFastWaves ? K_INSTR / kFastWaves : 1;  // loads per wave per tile
    static constexpr int NV = V_INSTR / kFastWaves;
    // K: 16 lanes read the same chunk of 16 consecutive rows; 256 bytes of banks hold 16 / KCPR rows
    static __device__ __forceinline__ int k_swz(int row) { return (row / (16 / KCPR)) & (KCPR - 1); }
    // V (transposed reads touch rows 4h + s, s = 0..3, 64 bytes each): spread s over the 64-byte windows
    static __device__ __forceinline__ int v_swz(int row) { return D == 128 ? 4 * (row & 3) : 4 * ((row >> 1) & 1); }
};

template <typename VT>
__device__ __forceinline__ typename PV<VT>::vec tr_pair(const unsigned char* p0, const unsigned char* p1) {
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)p0);
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)p1);
    const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(typename PV<VT>::vec, both);
}

// QB = 1: int8 Q and K with per-block scales (SageAttention).  QB = 2: Q and K in V's 16-bit type, one
// scale for the whole call (dense attention); in bytes a 16-bit K row of head_dim D is laid out, loaded
// and read exactly like an int8 row of head_dim 2 D.
// MASK: a bool mask tensor [B, Hq, M, N] (a byte per entry, non-zero = visible; rows 16-byte aligned and readable, as zeros, up to the next
// multiple of 16 keys: kv_len a multiple of 16, or rows the caller padded) on top of
// the key-hiding instance.  Every wave stages the 32 x 64 mask bytes of its own rows and step in a private slice
// of LDS (direct-to-LDS loads, three steps resident) and multiplies P by them.  The reference's arithmetic for
// rows that have not seen a visible key yet (scores of hidden keys are s - 1e6, not -inf:
// attn_qk_int8_per_block.py:46-52) and its skipping of 128 x 64 tiles without a visible key (:33-36) are
// served by the path that redoes a step: such rows start from the reference point -inf, which drives every
// step into that path until the row has seen a key.  a.mask_causal: the caller folded the causal mask into the
// tensor, so tiles beyond the causal limit of the workgroup's last row need no visit.  Additive masks and masks
// with unaligned rows stay with the general kernel (attn_fwd.hip).
//
// MT (the type of a mask entry): void = no mask tensor, bool = the bool mask above, _Float16 / __bf16 = an additive
// mask tensor in that storage type (attn_qk_int8_per_block.py:37-38,49-50: score + mask entry, no tile is skipped).
// Staged like the bool mask, 32 x 64 entries of 2 bytes per wave and step, two steps resident (with the four K/V
// tiles that fills the 160 KB of the CU at head_dim 128: the entries of step j + 1 are requested during the
// vector phase of step j, ahead of that phase's K/V loads, and waited for at the end of the matrix phase that
// follows).  The entry is added to the exponent of its score: fma(score, scale, entry - m).  Rows start from the
// reference point -inf like those of the bool instance, so the first step of every row runs the path that redoes a
// step, which takes the row maximum of score * scale + entry; so does a ragged last tile, whose keys past kv_len
// score -1e6 there as in the reference (mask entries read as -1e6, K as zeros).
// fp32 entries: 8 KB per wave and step, ONE step resident (two would not fit beside the K/V tiles): the entries of
// step j + 1 are requested at the end of the vector phase of step j, once its last entry has been read, and waited for
// at the end of the matrix phase that follows; the path that redoes a step reads its entries from memory again.
template <typename MT> struct MaskT { static constexpr int BYTES = sizeof(MT), SLOTS = sizeof(MT) == 4 ? 1 : 2; static constexpr bool ON = true, ADD = true; };
template <> struct MaskT<void> { static constexpr int BYTES = 1, SLOTS = 1; static constexpr bool ON = false, ADD = false; };
template <> struct MaskT<bool> { static constexpr int BYTES = 1, SLOTS = 3; static constexpr bool ON = true, ADD = false; };
constexpr float kMaskedScore = -1.0e6f;            // what the reference adds to the score of a hidden key

// an additive mask entry (16 bits, the low or the high half of a word) as fp32
template <typename MT> __device__ __forceinline__ float mask_entry(unsigned word, int hi);
template <> __device__ __forceinline__ float mask_entry<__bf16>(unsigned word, int hi) {
    return __builtin_bit_cast(float, hi ? (word & 0xffff0000u) : (word << 16));
}
template <> __device__ __forceinline__ float mask_entry<_Float16>(unsigned word, int hi) {
    return (float)__builtin_bit_cast(_Float16, (unsigned short)(hi ? (word >> 16) : (word & 0xffffu)));
}

template <int D, typename VT, bool CAUSAL, int QB, typename MT = void>
__global__ __launch_bounds__(kFastThreads, kFastWgPerCu) void sage_attn_fwd_fast_kernel(AttnArgs a, int nq2) {
    using F = FT<D, QB>;
    constexpr bool INT8 = QB == 1;
    constexpr bool MASK = MaskT<MT>::ON;         // a mask tensor is staged
    constexpr bool MADD = MaskT<MT>::ADD;        // ... an additive one (else bool)
    constexpr bool MF32 = MADD && MaskT<MT>::BYTES == 4;   // ... with fp32 entries (else 16-bit ones)
    constexpr int kMaskSlots = MaskT<MT>::SLOTS;                 // steps of mask entries resident per wave
    constexpr int kMaskWaveBytes = 32 * BN * MaskT<MT>::BYTES;   // 32 rows x 64 keys
    constexpr int kMaskInstr = kMaskWaveBytes / 1024;            // loads per wave and step
    constexpr int kMaskBytes = kMaskSlots * kFastWaves * kMaskWaveBytes;
    static_assert(!MASK || (CAUSAL && INT8), "the mask instances build on the key-hiding int8 instance");
    constexpr float BIAS = INT8 ? kBias : 0.0f;  // what the bits of a fresh score accumulator read as a float
    using PVT = PV<VT>;
    using vec16 = typename PVT::vec;
    constexpr float kSumLimit = sum_limit<VT>();
    __shared__ __attribute__((aligned(16))) unsigned char smem[F::TOTAL + (MASK ? kMaskBytes : 0)];


    // workgroup -> (batch, head, q-block); consecutive logical ids stay on one XCD (8 XCDs, round robin)
    // Under the causal flag a workgroup takes two q-blocks of its head, one after the other: block j (short
    // rows) and block nq2 - 1 - j (long rows), so that every workgroup of the launch runs about the same number
    // of steps (one q-block alone runs between 1/nq2 and all of them).  Short block first: the workgroups of a
    // head then start their long walks over the keys 4 steps apart, a window of tiles that stays in the XCD's L2;
    // with the long block first the short ones re-read the head's first tiles after they had been evicted
    // (1.35x the K/V bytes from memory at 8192 keys).
    int wg = blockIdx.x;
    if ((a.total_wg & 7) == 0) wg = (wg & 7) * (a.total_wg >> 3) + (wg >> 3);
    const bool paired = CAUSAL && a.causal;
    const int per_head = paired ? (nq2 + 1) / 2 : nq2;  // workgroups per (batch, head)
    // The keys of one (batch, head, q-block) may be split over `nsplit` workgroups (never under a mask tensor).  A
    // workgroup then sees the problem that starts at its first key: kv_len, the number of tiles and the causal
    // limits below all count from there, and its steps end where the next workgroup's begin.
    const int nsplit = MASK ? 1 : a.nsplit;
    const int split = wg % nsplit;
    wg /= nsplit;
    const int step0 = split * a.split_steps;  // first step of this workgroup's share of the keys
    const int kv_len = a.N - step0 * BN, nk = a.nk - step0;
    // heads that alternate within a q-block: measured to pay only under a mask with the causal mask folded in
    // (-7 %; +1..3 % for other shared masks, whose launches keep a head's q-blocks together for its K/V)
    const int ht = MASK && a.mask_causal ? a.head_tile : 1;
    const int jq = (wg / ht) % per_head;
    const int h = (wg / (ht * per_head)) % (a.Hq / ht) * ht + wg % ht;
    const int b = wg / (per_head * a.Hq);
    const int hk = h / a.groups;
  for (int pass = 0; pass < 2; pass++) {
    if (pass == 1 && (!paired || nq2 - 1 - jq == jq)) break;  // one q-block only, or the middle one of an odd count
    // Everything a pass needs is derived again from the thread index, made opaque here: values the compiler
    // would otherwise keep across the two passes cost registers the step loop cannot spare.
    int tid = threadIdx.x;
    asm volatile("" : "+v"(tid));
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int l32 = lane & 31;
    const int half = lane >> 5;
    // (a mask with the causal mask folded in: no pairs, the q-blocks with the most tiles are handed out first)
    const int iq = (paired && pass == 1) || (MASK && a.mask_causal) ? nq2 - 1 - jq : jq;
    const int m0 = iq * kFastRows;
    const int my_m = m0 + 32 * wave + l32;
    const bool row_ok = my_m < a.M;
    // The CAUSAL instance is the one that can hide keys: key n is visible to row m iff n <= lim(m), with
    // lim = min(m + kv_len - qo_len, kv_len - 1) under the causal flag and kv_len - 1 otherwise (a kv_len
    // that is not a multiple of 64 leaves hidden keys in the last tile).
    const int shift = kv_len - a.M;
    const int lim = !CAUSAL ? 0 : a.causal ? min(my_m + shift, kv_len - 1) : kv_len - 1;                  // this lane's row
    const int wlim = !CAUSAL ? 0 : a.causal ? min(m0 + 32 * wave + shift, kv_len - 1) : kv_len - 1;      // first row of the wave

    int nsteps = min(a.split_steps, nk);
    if (CAUSAL && (a.causal || (MASK && a.mask_causal))) {  // (a mask with the causal mask folded in: same bound)
        const int last_row = min(m0 + kFastRows, a.M) - 1;
        nsteps = max(min(nsteps, (last_row + shift + BN) / BN), 0);  // 0: no row of the workgroup sees a key (qo_len > kv_len)
    }

    // Q fragments: lane (row l32, half) holds bytes half * K_RS/2 + 16t .. +15 of its row for k-step t (any
    // order of the contraction index serves, as long as the K fragments use the same one)
    v4i qf[F::KSTEPS];
    {
        const int8_t* qp = a.q + ((int64_t)b * a.qs_b + (int64_t)h * a.qs_h + (int64_t)my_m * a.qs_n) * QB + half * (F::K_RS / 2);
#pragma unroll
        for (int t = 0; t < F::KSTEPS; t++)
            qf[t] = row_ok ? *reinterpret_cast<const v4i*>(qp + 16 * t) : v4i{0, 0, 0, 0};
    }
    const float qs = INT8 ? a.q_scale[((int64_t)b * a.Hq + h) * a.nq + min((kFastRows / BM) * iq + (wave >> 2), a.nq - 1)]
                          : a.qk_scale;
    // k_scale is read through the constant address space: the loads stay scalar (s_load_dword) even though
    // the loop contains assembly that clobbers memory, and they are tracked by lgkmcnt, not by the vmcnt
    // the direct-to-LDS loads are tracked with
    typedef __attribute__((address_space(4))) const float* const_f32_ptr;
    const const_f32_ptr ksp = (const_f32_ptr)(uintptr_t)(a.k_scale + ((int64_t)b * a.Hkv + hk) * a.nk + step0);
    auto step_scale = [&](int j, bool hides) {  // scale of the scores of step j (hides: the step may hold hidden keys)
        float s = INT8 ? qs * ksp[j] : qs;
        if (CAUSAL && hides) s = fmaxf(s, 1.17549435e-38f);  // keeps -inf * sc = -inf for hidden keys of an all-zero K block
        return s;
    };
    const int8_t* kg = a.k + ((int64_t)b * a.ks_b + (int64_t)hk * a.ks_h + (int64_t)step0 * BN * a.ks_n) * QB;
    const VT* vg = static_cast<const VT*>(a.v) + (int64_t)b * a.vs_b + (int64_t)hk * a.vs_h + (int64_t)step0 * BN * a.vs_n;

    // ---- staging: direct-to-LDS loads, 16 bytes per lane, 1 KB per wave instruction.  LDS piece
    //      p = 64 * instr + lane is chunk p % CPR of row p / CPR and receives the chunk (p % CPR) ^ swz(row)
    //      of that row from global memory.  Wave w issues instructions w, w + 8, ... of a tile (a K tile of
    //      head_dim 64 has only four, which waves 4-7 load a second time so that every wave has the same
    //      number of loads in flight).  The swizzle of a wave's piece does not depend on which of its
    //      instructions carries it (rows advance by a multiple of the swizzle period), so one per-lane
    //      byte offset serves all of them and the instruction index only moves the uniform base.
    static_assert(kFastWaves == 8 && F::V_INSTR % kFastWaves == 0, "load split");
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    const int k_idx = wave_u % F::K_INSTR;
    unsigned k_goff, v_goff;
    {
        const int pk = 64 * k_idx + lane, rk = pk / F::KCPR;
        k_goff = rk * (int)a.ks_n * QB + 16 * ((pk % F::KCPR) ^ F::k_swz(rk));
        const int pv = 64 * wave_u + lane, rv = pv / F::VCPR;
        v_goff = rv * (int)a.vs_n * 2 + 16 * ((pv % F::VCPR) ^ F::v_swz(rv));
    }
    static_assert((64 * kFastWaves / F::KCPR) % (16 / F::KCPR * F::KCPR) == 0 && (64 * kFastWaves / F::VCPR) % 4 == 0, "swizzle period");
    const int64_t k_instr_bytes = (int64_t)(64 * kFastWaves / F::KCPR) * a.ks_n * QB;  // rows per round of the waves * row stride
    const int64_t v_instr_bytes = (int64_t)(64 * kFastWaves / F::VCPR) * a.vs_n * 2;
    const unsigned lds0 = (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)smem;
    // The loads are written in assembly: the compiler would otherwise wait for every outstanding one
    // before each LDS read that follows.  Completion is tracked by hand with s_waitcnt vmcnt.
    // INVARIANT: m0 (the LDS address register of the load) is written here behind the compiler's back: it cannot be
    // named as a clobber.  That is sound only while the compiler itself never keeps a value in m0 in this kernel;
    // on gfx950 it would do so for s_movrel / v_movrel (registers indexed by a run-time value), LDS-direct and GWS
    // instructions and s_sendmsg, none of which this kernel gives it a reason to use (every register array is
    // indexed by compile-time constants).  tests/test_host_cpu.py compiles this file to assembly and fails if
    // anything but these moves mentions m0.
    auto dma16 = [](const unsigned char* base, unsigned voff, unsigned lds_addr) {
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                     :: "v"(voff), "s"(base), "s"(lds_addr) : "memory");
    };
    // The last tile of a kv_len that is not a multiple of 64 (CAUSAL instance only): rows past the end
    // re-read the last valid row (finite values under hidden scores), through per-lane offsets of their own.
    const bool ragged = CAUSAL && (kv_len % BN) != 0;
    unsigned k_goff_last[F::NK], v_goff_last[F::NV];
    if (CAUSAL) {
        const int last = (kv_len - 1) % BN;
#pragma unroll
        for (int e = 0; e < F::NK; e++) {
            const int pk = 64 * k_idx + lane, rk = pk / F::KCPR + e * (64 * kFastWaves / F::KCPR);
            k_goff_last[e] = min(rk, last) * (int)a.ks_n * QB + 16 * ((pk % F::KCPR) ^ F::k_swz(rk));
        }
#pragma unroll
        for (int e = 0; e < F::NV; e++) {
            const int pv = 64 * wave_u + lane, rv = pv / F::VCPR + e * (64 * kFastWaves / F::VCPR);
            v_goff_last[e] = min(rv, last) * (int)a.vs_n * 2 + 16 * ((pv % F::VCPR) ^ F::v_swz(rv));
        }
    }
    // unit e < NK of a wave's share of one K tile + one V tile: a K instruction; the rest: V instructions.
    // kt / vt: index of the tile behind ktile / vtile
    auto dma_unit = [&](auto ec, auto hc, int kbuf, const unsigned char* ktile, int kt, int vbuf, const unsigned char* vtile, int vt) {
        constexpr int e = decltype(ec)::value;
        constexpr bool HIDES = decltype(hc)::value;  // false: the caller knows that neither tile is a ragged last one
        if constexpr (e < F::NK) {
            const bool cut = HIDES && ragged && kt == nk - 1;
            dma16(cut ? ktile : ktile + e * k_instr_bytes, cut ? k_goff_last[e] : k_goff,
                  lds0 + kbuf * F::K_BYTES + 1024 * (k_idx + kFastWaves * e));
        } else {
            constexpr int ev = e - F::NK;
            const bool cut = HIDES && ragged && vt == nk - 1;
            dma16(cut ? vtile : vtile + ev * v_instr_bytes, cut ? v_goff_last[ev] : v_goff,
                  lds0 + F::V_BASE + vbuf * F::V_BYTES + 1024 * (wave_u + kFastWaves * ev));
        }
    };
    constexpr int NDMA = F::NK + F::NV + (MASK ? kMaskInstr : 0);  // loads per wave per step
    constexpr int NDMA_KV = F::NK + F::NV;

    // ---- mask staging (MASK): the wave's 32 rows x 64 keys of step t go to slot t % 3 of its own 2 KB slices, row
    //      after row (instruction e carries rows 16 e .. 16 e + 15, four lanes per row, so that neighbouring lanes
    //      read neighbouring bytes of memory).  Within a row the four 16-byte chunks are XOR-swizzled with bits 2-3
    //      of the row number: rows 4 apart, whose pieces would share banks, read different pieces.  Rows past
    //      qo_len re-read the last row, chunks past kv_len (last tile of a kv_len that is not a multiple of 64)
    //      the last chunk: duplicates of valid entries, so neither the products nor the look for a visible key see anything new.
    //      Additive 16-bit entries: 128 bytes per row, eight lanes per row, instruction e carries rows 8 e .. 8 e + 7;
    //      the eight chunks of a row are XOR-swizzled in pairs with bits 0-1 of the row number (a lane reads the two
    //      chunks of a 16-key slice with one instruction: they stay neighbours).
    const unsigned char* mask_row0 = nullptr;  // uniform: this wave's first mask row
    constexpr int MB = MaskT<MT>::BYTES;       // bytes per mask entry
    constexpr int kMaskLPR = BN * MB / 16;     // lanes (16-byte chunks) per staged row: 4 | 8
    unsigned m_goff[kMaskInstr] = {}, m_goff_last[kMaskInstr] = {};
    if constexpr (MASK) {
        const int row_first = min(m0 + 32 * wave_u, a.M - 1);
        mask_row0 = static_cast<const unsigned char*>(a.mask) + ((int64_t)b * a.ms_b + (int64_t)h * a.ms_h + (int64_t)row_first * a.ms_m) * MB;
        const int last_chunk = ((kv_len - 1) % BN) * MB / 16;
#pragma unroll
        for (int e = 0; e < kMaskInstr; e++) {
            const int rl = (64 / kMaskLPR) * e + lane / kMaskLPR;  // row of the wave's tile
            const int r = min(rl, a.M - 1 - row_first);
            const int chunk = MF32 ? (lane % kMaskLPR) ^ (rl & 7)
                            : MADD ? (lane % kMaskLPR) ^ (2 * (rl & 3))
                                   : (lane & 3) ^ ((lane >> 4) & 3);  // (bits 2-3 of the row number 16 e + lane / 4)
            m_goff[e] = (unsigned)((r * (int)a.ms_m) * MB + 16 * chunk);
            m_goff_last[e] = (unsigned)((r * (int)a.ms_m) * MB + 16 * min(chunk, last_chunk));
        }
    }
    auto dma_mask = [&](int tile, int slot) {
        if constexpr (MASK) {
            const bool cut = ragged && tile == nk - 1;
#pragma unroll
            for (int e = 0; e < kMaskInstr; e++)
                dma16(mask_row0 + (int64_t)tile * BN * MB, cut ? m_goff_last[e] : m_goff[e],
                      lds0 + F::TOTAL + (slot * kFastWaves + wave_u) * kMaskWaveBytes + 1024 * e);
        }
    };
    // (additive) the lane's entries of 16-key slice tp of a staged step: four words, the entries of score registers
    // 8 (tp & 1) + 0 .. 3 (two words) and + 4 .. 7 (two words) of tile tp >> 1
    // (fp32 entries) 256 bytes per staged row, sixteen lanes per row, instruction e carries rows 4 e .. 4 e + 3; the
    // sixteen chunks of a row are XOR-swizzled with bits 0-2 of the row number.  mask_half: the lane's four entries of
    // half-slice hs = 2 tp + j (score registers 8 (tp & 1) + 4 j .. + 3 of tile tp >> 1): chunk 2 hs + half of its row.
    auto mask_half = [&](int hs, v4f& e) {
        const unsigned char* row = smem + F::TOTAL + wave * kMaskWaveBytes + l32 * (BN * MB);
        e = *reinterpret_cast<const v4f*>(row + ((32 * hs) ^ (16 * ((l32 & 7) ^ half))));
    };
    // the same four entries from memory (the path that redoes a step: the staged ones may have been replaced by then)
    auto mask_half_global = [&](int n_first, int hs, v4f& e) {
        const int64_t row = min(my_m, a.M - 1);
        const float* rp = static_cast<const float*>(a.mask) + (int64_t)b * a.ms_b + (int64_t)h * a.ms_h + row * a.ms_m;
        const int key = min(n_first + 8 * hs + 4 * half, ((a.N - 1) / 4) * 4);  // (keys past kv_len: any readable entry, unused)
        e = *reinterpret_cast<const v4f*>(rp + key);
    };
    auto mask_entries = [&](int slot, int tp, unsigned (&w)[4]) {
        const unsigned char* row = smem + F::TOTAL + (slot * kFastWaves + wave) * kMaskWaveBytes + l32 * (BN * MB) + 8 * half;
        const v2u* piece = reinterpret_cast<const v2u*>(row + 32 * (tp ^ (l32 & 3)));
        const v2u lo = piece[0], hi = piece[2];
        w[0] = lo[0]; w[1] = lo[1]; w[2] = hi[0]; w[3] = hi[1];
    };
    // The lane's mask bytes of 16-key slice tp of a staged step: two words, keys 8 g + 4 half .. + 3 for the even and
    // the odd g of the slice (the keys of score registers 8 (tp & 1) .. + 3 and + 4 .. + 7 of tile tp >> 1).
    auto mask_words = [&](int slot, int tp, unsigned& even, unsigned& odd) {
        const unsigned char* row = smem + F::TOTAL + (slot * kFastWaves + wave) * kMaskWaveBytes + l32 * BN + 4 * half;
        const unsigned* piece = reinterpret_cast<const unsigned*>(row + ((16 * tp) ^ (4 * (l32 & 12))));
        even = piece[0];
        odd = piece[2];
    };
    // Does the current step's mask tile hold a visible key for this wave's 128-row block?  (The reference skips a
    // 128 x 64 tile whose mask is False everywhere, attn_qk_int8_per_block.py:33-36.)  Only the path that redoes a
    // step asks: rows that have seen a key need no answer, their P of a hidden key is 0 either way.  The four
    // slices of the block lie side by side in the slot; all of them landed before the barrier that opened the
    // previous phase and are refilled two phases from now at the earliest.
    auto tile_has_visible_key = [&](int slot) {
        const uint4* blk = reinterpret_cast<const uint4*>(smem + F::TOTAL + (slot * kFastWaves + 4 * (wave >> 2)) * kMaskWaveBytes);
        unsigned any = 0;
#pragma unroll
        for (int k = 0; k < 4 * kMaskWaveBytes / (64 * 16); k++) {
            const uint4 w = blk[lane + 64 * k];
            any |= w.x | w.y | w.z | w.w;
        }
        return __builtin_amdgcn_ballot_w64(any != 0) != 0;
    };
    // ---- fragment read offsets (undoing the swizzle)
    // K: lane (row l32, half) reads chunk half * K_RS/32 + t of its row for k-step t
    int kf_off[F::KSTEPS];
#pragma unroll
    for (int t = 0; t < F::KSTEPS; t++) kf_off[t] = l32 * F::K_RS + 16 * ((half * (F::K_RS / 32) + t) ^ F::k_swz(l32));
    // V, ds_read_b64_tr_b16: in each group of 16 lanes, lane 4s+a supplies keys row s, channels 4a..4a+3,
    // and lane i receives channel i of the four rows.  Groups: (channels 0-15 | 16-31) x (half 0 | 1).
    int vtr_off[F::DTILES];
    {
        const int s4 = (lane >> 2) & 3, a4 = lane & 3, g1 = (lane >> 4) & 1;
#pragma unroll
        for (int dt = 0; dt < F::DTILES; dt++)
            vtr_off[dt] = (4 * half + s4) * F::V_RS + 16 * ((4 * dt + 2 * g1 + (a4 >> 1)) ^ F::v_swz(s4)) + 8 * (a4 & 1);
    }

    // The int32 accumulators start from the bit pattern of the float 1.5 * 2^23: since |dot| < 2^22,
    // accumulator bits reinterpreted as fp32 ARE kBias + dot, so no int -> float conversion is needed.
    // (16-bit Q and K: fp32 accumulators that start from zero, kept in the same registers as bits.)
    v16i bias16;
#pragma unroll
    for (int i = 0; i < 16; i++) {
        int b;  // materialised once through an opaque move, so the block stays in VGPRs for the whole kernel
        asm volatile("v_mov_b32 %0, %1" : "=v"(b) : "s"(INT8 ? kBiasBits : 0));
        bias16[i] = b;
    }
    // Row sums of P by the matrix core: one 16x16x32 instruction per 16-key slice multiplies a 0/1 pattern
    // with the slice's P^T registers as they are.  Read as a 32 x 16 B operand, those registers hold four
    // groups of eight keys: (rows 0-15 | rows 16-31) x (keys 0-7 | keys 8-15) of the slice; output rows
    // 0-3 and 8-11 add the two groups of rows 0-15, output rows 4-7 and 12-15 those of rows 16-31, which
    // is where the lanes that own those query rows read their results.  Every lane ends up with the sum
    // over all 16 keys of its own row (both halves), in four equal registers.
    vec16 sum_pattern;
    {
        const VT c = (((lane >> 4) & 1) == ((lane >> 2) & 1)) ? (VT)1.0f : (VT)0.0f;
#pragma unroll
        for (int e = 0; e < 8; e++) sum_pattern[e] = c;
    }
    auto qk_mfma = [](v4i kf, v4i q, v16i acc) {
        if constexpr (INT8) {
            return __builtin_amdgcn_mfma_i32_32x32x32_i8(kf, q, acc, 0, 0, 0);
        } else {
            return __builtin_bit_cast(v16i, PVT::mfma(__builtin_bit_cast(vec16, kf), __builtin_bit_cast(vec16, q),
                                                      __builtin_bit_cast(v16f, acc)));
        }
    };
    auto qk_tile = [&](const unsigned char* kbase, int kt) {
        v16i acc = bias16;
#pragma unroll
        for (int t = 0; t < F::KSTEPS; t++) {
            const v4i kf = *reinterpret_cast<const v4i*>(kbase + kf_off[t] + 32 * kt * F::K_RS);
            acc = qk_mfma(kf, qf[t], acc);
        }
        return acc;
    };

    float m_i;         // reference point of the row's exponentials: set from the first tile below
    float l_i = 0.0f;  // (the reference's initial l = 1 is multiplied by exp2(-inf) = 0 in its first step)
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
    constexpr int DEFER = (D == 64 && INT8 && !MF32) ? 4 : 0;  // exponential units moved into the MFMA phase (measured per instance;
                                                               // fp32 mask entries: every unit reads them before the slot is refilled)
    constexpr bool kWholeRowSums = QB == 2 && !CAUSAL;      // row sums by the matrix core: every lane holds its whole row's sum
    constexpr int KDIST = 4 < QK_SLOTS ? 4 : QK_SLOTS;      // K fragments in flight
    constexpr int VDIST = 3 < QK_SLOTS ? 3 : QK_SLOTS - 1;  // V fragments in flight
    static_assert(KDIST <= QK_SLOTS && VDIST < QK_SLOTS && 16 % QK_SLOTS == 0, "slot plan");
    static_assert(DEFER <= QK_SLOTS, "every P of a step exists when its row sums are checked, before the first P.V");

    // Scores live in two register sets that swap roles every step (the loop body is instantiated
    // for both parities), so the accumulators Q.K^T writes in one iteration are read in place by
    // the exponentials of the next one.
    v16i sbuf[2][2];  // [parity][32-key tile]: int32 accumulators whose bits are the float kBias + dot
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
                x[e] = (n > lim) ? -INFINITY : x[e];
                sbuf[P][kt][i] = __builtin_bit_cast(int, x[e]);
            }
        }
        acc = fmaxf(fmaxf(acc, x[0]), x[1]);
        acc = fmaxf(fmaxf(acc, x[2]), x[3]);
        asm volatile("" ::"v"(acc));  // pin to this slot (otherwise sunk below the matrix instructions)
    };
    // The two lanes that share a row (l32 and l32 + 32) agree on the larger of their values.
    auto row_pair_max = [](float x) {
        const v2u sw = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(unsigned, x), __builtin_bit_cast(unsigned, x), false, false);
        const unsigned mine = sw[0], other = sw[1];  // (scalar copies: bit_cast of a vector element lvalue reads element 0)
        return fmaxf(__builtin_bit_cast(float, mine), __builtin_bit_cast(float, other));
    };

    // ---- prologue: K0, K1, K2, V0, V1 in LDS; scores of step 0 in registers.  Tile indices past the
    //      last step are clamped to it: such a tile is fetched again into a buffer nobody reads.
    const int64_t k_tile_bytes = (int64_t)BN * a.ks_n * QB, v_tile_bytes = (int64_t)BN * a.vs_n * 2;
    const unsigned char* k_fetch = reinterpret_cast<const unsigned char*>(kg);
    const unsigned char* v_fetch = reinterpret_cast<const unsigned char*>(vg);
    int k_tile = 0, v_tile = 0;  // indices of the tiles behind k_fetch / v_fetch
    sfor<NDMA_KV>([&](auto ec) { dma_unit(ec, IC<1>{}, 0, k_fetch, k_tile, 0, v_fetch, v_tile); });
    if (nsteps > 1) { k_fetch += k_tile_bytes; v_fetch += v_tile_bytes; k_tile++; v_tile++; }
    sfor<NDMA_KV>([&](auto ec) { dma_unit(ec, IC<1>{}, 1, k_fetch, k_tile, 1, v_fetch, v_tile); });
    if (nsteps > 2) { k_fetch += k_tile_bytes; v_fetch += v_tile_bytes; k_tile++; v_tile++; }
    sfor<F::NK>([&](auto ec) { dma_unit(ec, IC<1>{}, 2, k_fetch, k_tile, 2, v_fetch, v_tile); });
    // from here on k_fetch / v_fetch point at the tiles fetched during step 0: K of step 3, V of step 2
    if (nsteps > 3) { k_fetch += k_tile_bytes; k_tile++; }
    dma_mask(0, 0);
    if constexpr (kMaskSlots == 3) dma_mask(max(min(1, nsteps - 1), 0), 1);  // (nsteps = 0: a workgroup that sees no key; tile 0 exists all the same)
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the direct-to-LDS loads have landed
    __syncthreads();
    sbuf[0][0] = qk_tile(smem, 0);
    sbuf[0][1] = qk_tile(smem, 1);
    sc = step_scale(0, true);
    {   // the row maximum of the first tile is the reference point the row starts from
        float raw_max = -INFINITY;
        const bool masked0 = CAUSAL && (BN - 1 > wlim);
        sfor<8>([&](auto uc) { head_unit(IC<0>{}, uc, 0, masked0, raw_max); });
        // (a row that sees no key at all, qo_len > kv_len under the causal flag, keeps a finite reference
        // point: its exponentials are then exp2(-inf) = 0 and it ends with l = 0)
        m_i = fmaxf((row_pair_max(raw_max) - BIAS) * sc, -1.0e30f);
        if (MASK && !MADD) m_i = -INFINITY;  // no visible key seen yet: the first step with one sets the reference point
        if constexpr (MADD) {  // the maximum of score * scale + entry over the first tile (its entries are staged)
            float mx = -INFINITY;
            sfor<4>([&](auto tc) {
                constexpr int tp = decltype(tc)::value, kt = tp >> 1;
                float e8[8];
                if constexpr (MF32) {
                    v4f lo, hi;
                    mask_half(2 * tp, lo);
                    mask_half(2 * tp + 1, hi);
#pragma unroll
                    for (int c = 0; c < 4; c++) { e8[c] = lo[c]; e8[4 + c] = hi[c]; }
                } else {
                    unsigned w4[4];
                    mask_entries(0, tp, w4);
#pragma unroll
                    for (int c = 0; c < 8; c++) e8[c] = mask_entry<MT>(w4[c >> 1], c & 1);
                }
#pragma unroll
                for (int c = 0; c < 8; c++) {
                    const int bits = sbuf[0][kt][8 * (tp & 1) + c];
                    mx = fmaxf(mx, __builtin_fmaf(as_f(bits) - BIAS, sc, e8[c]));
                }
            });
            m_i = fmaxf(row_pair_max(mx), -1.0e30f);
        }
    }
    int mslot = 0;  // slot of the current step's mask bytes (step % 3)

    // ---- one step.  Each wave alternates a VALU phase (exponentials of its step) and an MFMA phase
    // (Q.K^T of the next step, P.V of this one, with the row sums in the shadow of the matrix
    // instructions); the two waves that share a SIMD run half a step
    // apart (see the barrier before the loop), so one feeds the matrix core while the other
    // occupies the VALU.  Two barriers per step.
    // HIDES = false is the body for steps that hide no key of this step or the next and fetch no ragged tile:
    // the code of the instance that cannot hide keys at all.  Both bodies pass the same two barriers, so the
    // waves of a workgroup may be in different ones.
    auto body = [&](auto pc, auto hc, int step) {
        constexpr int P = decltype(pc)::value;  // == step & 1
        constexpr bool HIDES = CAUSAL && decltype(hc)::value;
        // tile t of K (of V) lives in LDS buffer t % 4: this step reads K of step+1 and V of step, and
        // fetches K of step+3 and V of step+2 into the buffers that K of step-1 and V of step-2 left
        int kaddr[F::KSTEPS], vaddr[F::DTILES];
#pragma unroll
        for (int t = 0; t < F::KSTEPS; t++) {
            kaddr[t] = kf_off[t] + ((step + 1) & 3) * F::K_BYTES;
            asm volatile("" : "+v"(kaddr[t]));  // computed once per step, here in the VALU phase
        }
#pragma unroll
        for (int dt = 0; dt < F::DTILES; dt++) {
            vaddr[dt] = vtr_off[dt] + F::V_BASE + (step & 3) * F::V_BYTES;
            asm volatile("" : "+v"(vaddr[dt]));
        }
        v4i kfr[QK_SLOTS];
        vec16 vfr[PV_SLOTS];
        auto read_k = [&](auto ic) {
            constexpr int i = decltype(ic)::value;
            kfr[i] = *reinterpret_cast<const v4i*>(smem + kaddr[i / 2] + 32 * (i % 2) * F::K_RS);
        };
        auto read_v = [&](auto jc) {
            constexpr int j = decltype(jc)::value;
            const unsigned char* p0 = smem + vaddr[j % F::DTILES] + 16 * (j / F::DTILES) * F::V_RS;
            vfr[j] = tr_pair<VT>(p0, p0 + 8 * F::V_RS);
        };
        const int n0 = step * BN;
        const bool live = step < nsteps;  // false only for the padding step after an odd number of steps

        // ===== VALU phase: exponentials of this step (scores in sbuf[P]) =====
        // No row maximum is taken: the exponentials use the reference point m_i the row already has, which
        // any value not far below the true maximum serves equally well (the result is O / l either way).
        // Should it make a P too large, the row sums show it before the first P.V instruction, and the step
        // is redone against its true maximum: see redo_if_large below.
        float neg_m;
        const bool folded = !INT8 || kBias * sc < kBiasFoldLimit;
        if (!folded) {
#pragma unroll
            for (int kt = 0; kt < 2; kt++)
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const int bits = sbuf[P][kt][i];
                    sbuf[P][kt][i] = __builtin_bit_cast(int, as_f(bits) - kBias);
                }
        }
        neg_m = folded ? __builtin_fmaf(-BIAS, sc, -m_i) : -m_i;
        if (!live) neg_m = -INFINITY;  // padding step: every P is exp2(-inf) = 0

        // The direct-to-LDS loads are issued from the VALU phase, where a stalled issue delays no matrix
        // instruction.
        const int mslot_next = mslot == kMaskSlots - 1 ? 0 : mslot + 1;
        // (additive: the entries of step + 1, into the slot that step - 1 left; ahead of the K/V loads, because they
        // are the ones waited for first: at the end of the coming matrix phase)
        if constexpr (MADD && !MF32) dma_mask(min(step + 1, nsteps - 1), mslot_next);
        sfor<NDMA_KV>([&](auto ec) { dma_unit(ec, IC<HIDES>{}, (step + 3) & 3, k_fetch, k_tile, (step + 2) & 3, v_fetch, v_tile); });
        if constexpr (MASK && !MADD) dma_mask(min(step + 2, nsteps - 1), mslot_next == kMaskSlots - 1 ? 0 : mslot_next + 1);  // the mask bytes of step + 2
        vec16 pf[4];
        float lsum = 0.0f;
        const float sc_e = sc;  // this step's scale (sc moves on to the next step below)
        unsigned mw[2][2] = {{0, 0}, {0, 0}};  // (bool mask) the lane's mask bytes of the 16-key slice in work and of the next one
        unsigned me[2][4] = {};                // (additive 16-bit mask) the lane's entries of the slice in work and of the next one
        v4f mf[2] = {};                        // (additive fp32 mask) the lane's entries of the half-slice in work and of the next one
        if constexpr (MASK && !MADD) mask_words(mslot, 0, mw[0][0], mw[0][1]);
        if constexpr (MADD && !MF32) mask_entries(mslot, 0, me[0]);
        if constexpr (MF32) mask_half(0, mf[0]);
        auto exp_unit = [&](auto uc) {  // two scores -> two 16-bit P values
            constexpr int u = decltype(uc)::value;
            constexpr int tp = u >> 2, w = u & 3, kt = tp >> 1, i0 = 8 * (tp & 1) + 2 * w;
            const int b0 = sbuf[P][kt][i0], b1 = sbuf[P][kt][i0 + 1];
            float t0 = neg_m, t1 = neg_m;
            if constexpr (MF32) {  // the mask entry joins the exponent: score * scale + entry - m
                constexpr int hs = 2 * tp + (w >> 1);
                if constexpr ((w & 1) == 0 && hs < 7) mask_half(hs + 1, mf[(hs + 1) & 1]);
                t0 += mf[hs & 1][2 * (w & 1)];
                t1 += mf[hs & 1][2 * (w & 1) + 1];
            } else if constexpr (MADD) {
                if constexpr (w == 0 && tp < 3) mask_entries(mslot, tp + 1, me[(tp + 1) & 1]);
                const unsigned word = me[tp & 1][w];
                t0 += mask_entry<MT>(word, 0);
                t1 += mask_entry<MT>(word, 1);
            }
            float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(as_f(b0), sc_e, t0));
            float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(as_f(b1), sc_e, t1));
            if constexpr (MASK && !MADD) {
                // P of a hidden key is 0.  An overflowed P times 0 is NaN: the row sum then
                // sends the step into the path that redoes it.
                if constexpr (w == 0 && tp < 3) mask_words(mslot, tp + 1, mw[(tp + 1) & 1][0], mw[(tp + 1) & 1][1]);
                // (any non-zero byte keeps the key: the conversion clamps to [0, 1], an output modifier of the same
                // instruction)
                const unsigned word = mw[tp & 1][w >> 1];
                p0 *= __builtin_amdgcn_fmed3f((float)((word >> (16 * (w & 1))) & 0xffu), 0.0f, 1.0f);
                p1 *= __builtin_amdgcn_fmed3f((float)((word >> (16 * (w & 1) + 8)) & 0xffu), 0.0f, 1.0f);
            }
            pf[tp][2 * w] = (VT)p0;
            pf[tp][2 * w + 1] = (VT)p1;
        };
        // The last DEFER of the 16 units wait for the MFMA phase (head_dim 64: that phase has half the
        // matrix instructions, so it takes a share of the exponentials to keep the two phases even).
        // Where the row sums are taken is a measured choice per instance: in the shadow of the Q.K^T
        // instructions everywhere (head_dim 128, int8: 10 % faster than here; 16-bit without hidden keys:
        // 4 %), except in the 16-bit instance that hides keys, whose MFMA phase is the longer one (32 matrix
        // instructions and the masking of the diagonal tiles): there they follow their exponentials (-4.5 %).
        constexpr bool kSumsEarly = QB == 2 && CAUSAL && DEFER == 0;
        sfor<16 - DEFER>([&](auto uc) {
            constexpr int u = decltype(uc)::value;
            exp_unit(uc);
            if constexpr (kSumsEarly && u >= 2) lsum = PVT::dot2_ones(pf[(u - 2) >> 2], (u - 2) & 3, lsum);
        });
        if constexpr (kSumsEarly) {
            lsum = PVT::dot2_ones(pf[3], 2, lsum);
            lsum = PVT::dot2_ones(pf[3], 3, lsum);
        }
        // (fp32 mask entries: the last one of this step has been read; the one slot takes those of the next step)
        if constexpr (MF32) dma_mask(min(step + 1, nsteps - 1), 0);
        // A lane's 32 P of a step sum to less than kSumLimit, or the step is redone: so no P overflows the
        // 16-bit type (nor does a sum or a product with V come near the fp32 range), and a row whose scores
        // rise keeps its reference point within log2(kSumLimit) of its maximum.  Wave-wide decision; rare
        // after the first steps of a row (the maximum of a row rises ever more slowly).
        // The sums are complete SUM_SLOTS matrix instructions into the phase; the wave vote on them is taken
        // there and only tested before the first P.V instruction, four matrix instructions later, so that
        // neither the last sum nor the compare is waited for (2-3 % on the causal and the 16-bit instances).
        // ... and in the 16-bit instance without hidden keys the matrix core takes them (sum_pattern above): four
        // cheap matrix instructions instead of 16 v_dot2 on an issue port that the 32 matrix instructions of
        // its step already load (-5 %; neutral for the int8 instances, which keep v_dot2 and half-row sums).
        constexpr bool kMfmaSums = kWholeRowSums;
        constexpr int SUM_SLOTS = kSumsEarly ? -1 : (DEFER == 0 && QK_SLOTS >= 8) ? QK_SLOTS - 4 : QK_SLOTS;
        v4f sum4 = {0.0f, 0.0f, 0.0f, 0.0f};
        unsigned long long large = 0;
        auto redo_if_large = [&]() {
            if constexpr (MADD) {
                // a ragged last tile always comes here: its keys past kv_len score -1e6 (the reference reads their
                // mask entries as -1e6 and their K as zeros), which only this path accounts for
                if (large != 0 || (ragged && step == nk - 1)) {
                    float raw = -INFINITY;
                    float past_end = 0.0f;  // number of the lane's keys of this step that lie past kv_len
                    sfor<4>([&](auto tc) {
                        constexpr int tp = decltype(tc)::value, kt = tp >> 1;
                        float e8[8];
                        if constexpr (MF32) {
                            v4f lo, hi;
                            mask_half_global(n0, 2 * tp, lo);
                            mask_half_global(n0, 2 * tp + 1, hi);
#pragma unroll
                            for (int c = 0; c < 4; c++) { e8[c] = lo[c]; e8[4 + c] = hi[c]; }
                        } else {
                            unsigned w4[4];
                            mask_entries(mslot, tp, w4);
#pragma unroll
                            for (int c = 0; c < 8; c++) e8[c] = mask_entry<MT>(w4[c >> 1], c & 1);
                        }
#pragma unroll
                        for (int c = 0; c < 8; c++) {
                            const int i = 8 * (tp & 1) + c;
                            const int bits = sbuf[P][kt][i];
                            const float x = as_f(bits);
                            float sv = __builtin_fmaf(folded ? x - BIAS : x, sc_e, e8[c]);
                            if (x == -INFINITY) {  // past kv_len
                                sv = -INFINITY;
                                past_end += 1.0f;
                            }
                            sbuf[P][kt][i] = __builtin_bit_cast(int, sv);
                            raw = fmaxf(raw, sv);
                        }
                    });
                    if (past_end > 0.0f) raw = fmaxf(raw, kMaskedScore);
                    const float m_new = fmaxf(m_i, row_pair_max(raw));
                    const float alpha = __builtin_amdgcn_exp2f(m_i - m_new);  // 0 for a row that had no reference point yet
                    l_i *= alpha;
                    m_i = m_new;
#pragma unroll
                    for (int dt = 0; dt < F::DTILES; dt++)
#pragma unroll
                        for (int i = 0; i < 16; i++) o[dt][i] *= alpha;
                    lsum = 0.0f;
                    sfor<16>([&](auto uc) {
                        constexpr int u = decltype(uc)::value;
                        constexpr int tp = u >> 2, w = u & 3, kt = tp >> 1, i0 = 8 * (tp & 1) + 2 * w;
                        const int b0 = sbuf[P][kt][i0], b1 = sbuf[P][kt][i0 + 1];
                        pf[tp][2 * w] = (VT)__builtin_amdgcn_exp2f(as_f(b0) - m_i);
                        pf[tp][2 * w + 1] = (VT)__builtin_amdgcn_exp2f(as_f(b1) - m_i);
                        lsum = PVT::dot2_ones(pf[tp], w, lsum);
                    });
                    lsum = __builtin_fmaf(past_end, __builtin_amdgcn_exp2f(kMaskedScore - m_i), lsum);
                }
                return;
            }
            if constexpr (MASK) {
                if (large != 0 && !tile_has_visible_key(mslot)) {
                    // no visible key for this 128-row block in this tile: the reference skips it.  (Rows without a
                    // reference point get here every step until they see a key: their P came out inf or NaN.)
#pragma unroll
                    for (int tp = 0; tp < 4; tp++)
#pragma unroll
                        for (int c = 0; c < 8; c++) pf[tp][c] = (VT)0.0f;
                    lsum = 0.0f;
                } else if (large != 0) {
                    // The reference's own arithmetic (attn_qk_int8_per_block.py:44-62): score = dot * scale, plus -1e6
                    // where the mask hides the key; a key past kv_len scores exactly -1e6 (K and the mask are read
                    // as zeros / False there).
                    // (Its V rows are zeros too: such a key adds exp2(-1e6 - m) to the row sum and nothing to O; here
                    // its P stays 0 and the row sum gets the term directly.)
                    float raw = -INFINITY;
                    float past_end = 0.0f;  // number of the lane's keys of this step that lie past kv_len
                    sfor<4>([&](auto tc) {
                        constexpr int tp = decltype(tc)::value, kt = tp >> 1;
                        unsigned ev, od;
                        mask_words(mslot, tp, ev, od);
#pragma unroll
                        for (int c = 0; c < 8; c++) {
                            const int i = 8 * (tp & 1) + c;
                            const int bits = sbuf[P][kt][i];
                            const float x = as_f(bits);
                            const unsigned keep = (((c >> 2) ? od : ev) >> (8 * (c & 3))) & 0xffu;
                            float sv = __builtin_fmaf(folded ? x - BIAS : x, sc_e, keep ? 0.0f : kMaskedScore);
                            if (x == -INFINITY) {  // hidden by position, not by the mask: past kv_len
                                sv = -INFINITY;
                                past_end += 1.0f;
                            }
                            sbuf[P][kt][i] = __builtin_bit_cast(int, sv);
                            raw = fmaxf(raw, sv);
                        }
                    });
                    if (past_end > 0.0f) raw = fmaxf(raw, kMaskedScore);
                    const float m_new = fmaxf(m_i, row_pair_max(raw));
                    const float alpha = __builtin_amdgcn_exp2f(m_i - m_new);  // 0 for a row that had no reference point yet
                    l_i *= alpha;
                    m_i = m_new;
#pragma unroll
                    for (int dt = 0; dt < F::DTILES; dt++)
#pragma unroll
                        for (int i = 0; i < 16; i++) o[dt][i] *= alpha;
                    lsum = 0.0f;
                    sfor<16>([&](auto uc) {
                        constexpr int u = decltype(uc)::value;
                        constexpr int tp = u >> 2, w = u & 3, kt = tp >> 1, i0 = 8 * (tp & 1) + 2 * w;
                        const int b0 = sbuf[P][kt][i0], b1 = sbuf[P][kt][i0 + 1];
                        pf[tp][2 * w] = (VT)__builtin_amdgcn_exp2f(as_f(b0) - m_i);
                        pf[tp][2 * w + 1] = (VT)__builtin_amdgcn_exp2f(as_f(b1) - m_i);
                        lsum = PVT::dot2_ones(pf[tp], w, lsum);
                    });
                    lsum = __builtin_fmaf(past_end, __builtin_amdgcn_exp2f(kMaskedScore - m_i), lsum);
                }
                return;
            }
            if (large != 0) {
                float raw = -INFINITY;
#pragma unroll
                for (int kt = 0; kt < 2; kt++)
#pragma unroll
                    for (int i = 0; i < 16; i++) {
                        const int bits = sbuf[P][kt][i];
                        raw = fmaxf(raw, as_f(bits));
                    }
                const float rmax = (row_pair_max(raw) - (folded ? BIAS : 0.0f)) * sc_e;
                const float m_new = fmaxf(m_i, rmax);
                const float alpha = __builtin_amdgcn_exp2f(m_i - m_new);
                l_i *= alpha;
                m_i = m_new;
#pragma unroll
                for (int dt = 0; dt < F::DTILES; dt++)
#pragma unroll
                    for (int i = 0; i < 16; i++) o[dt][i] *= alpha;
                neg_m = folded ? __builtin_fmaf(-BIAS, sc_e, -m_i) : -m_i;
                lsum = 0.0f;
                sfor<16>([&](auto uc) {
                    constexpr int u = decltype(uc)::value;
                    exp_unit(uc);
                    lsum = PVT::dot2_ones(pf[u >> 2], u & 3, lsum);
                });
                if constexpr (kMfmaSums) lsum += __shfl_xor(lsum, 32);  // this instance keeps whole-row sums in every lane
            }
        };
        if constexpr (kSumsEarly) large = __builtin_amdgcn_ballot_w64(!(lsum < kSumLimit));
        sc = step_scale(min(step + 1, nsteps - 1), HIDES);
        __builtin_amdgcn_sched_barrier(0);
        // The first K fragments of the coming MFMA phase are requested before the barrier (their tile
        // landed a step ago), so the phase does not open with an LDS round trip.
        sfor<KDIST>(read_k);
        __builtin_amdgcn_sched_barrier(0);
        // The loads issued in the previous VALU phase have landed (all but the NDMA just issued): the
        // tiles they belong to are first read two barriers from here.
        __builtin_amdgcn_s_waitcnt(0x0F70 | NDMA);
        __builtin_amdgcn_s_barrier();        // phase switch: this wave takes the matrix core
        __builtin_amdgcn_sched_barrier(0);

        // ===== MFMA phase =====
        __builtin_amdgcn_s_setprio(1);
        const bool masked_n = HIDES && (n0 + 2 * BN - 1 > wlim);
        sfor<NSLOTS>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            if constexpr (i < QK_SLOTS) {
                constexpr int kt = i % 2, t = i / 2;  // alternate the two accumulation chains
                if constexpr (t == 0) {
                    sbuf[1 - P][kt] = qk_mfma(kfr[i], qf[t], bias16);
                } else {
                    sbuf[1 - P][kt] = qk_mfma(kfr[i], qf[t], sbuf[1 - P][kt]);
                }
                if constexpr (i + KDIST < QK_SLOTS) read_k(IC<i + KDIST>{});
                if constexpr (i >= QK_SLOTS - VDIST) read_v(IC<i - (QK_SLOTS - VDIST)>{});
                // row sums of P ride in the shadow of the Q.K^T instructions
                if constexpr (kMfmaSums) {
                    if constexpr (i < 4) {  // one per slot, behind the first four Q.K^T instructions
                        if constexpr (i == 0) sum4 = PVT::mfma16(sum_pattern, pf[0], v4f{0.0f, 0.0f, 0.0f, 0.0f});
                        else sum4 = PVT::mfma16(sum_pattern, pf[i], sum4);
                    }
                    if constexpr (i == QK_SLOTS - 2) {  // the four sum instructions have long finished
                        lsum = sum4[0];
                        large = __builtin_amdgcn_ballot_w64(!(lsum < kSumLimit));  // also set for inf and NaN
                        asm volatile("" ::"s"(large));
                    }
                } else {
                    sfor<16 - DEFER>([&](auto rc) {
                        constexpr int u = decltype(rc)::value;
                        if constexpr (!kSumsEarly && u * SUM_SLOTS / (16 - DEFER) == i) {
                            lsum = PVT::dot2_ones(pf[u >> 2], u & 3, lsum);
                            asm volatile("" ::"v"(lsum));
                        }
                    });
                }
                if constexpr (!kMfmaSums && i == SUM_SLOTS - 1 && SUM_SLOTS < QK_SLOTS) {
                    large = __builtin_amdgcn_ballot_w64(!(lsum < kSumLimit));  // also set for inf and NaN
                    asm volatile("" ::"s"(large));
                }
            } else {
                constexpr int j = i - QK_SLOTS, tp = j / F::DTILES, dt = j % F::DTILES;
                if constexpr (j == 0) {
                    if constexpr (!kSumsEarly && SUM_SLOTS == QK_SLOTS) large = __builtin_amdgcn_ballot_w64(!(lsum < kSumLimit));
                    redo_if_large();
                    __builtin_amdgcn_sched_barrier(0);
                }
                o[dt] = PVT::mfma(vfr[j], pf[tp], o[dt]);
                if constexpr (j + VDIST < PV_SLOTS) read_v(IC<j + VDIST>{});
                // hidden keys of the next step's scores (Q.K^T finished above) are set to -inf under the
                // P.V instructions
                if constexpr (HIDES) {
                    sfor<8 / PV_SLOTS + (8 % PV_SLOTS != 0)>([&](auto rc) {
                        constexpr int u = j * (8 / PV_SLOTS + (8 % PV_SLOTS != 0)) + decltype(rc)::value;
                        if constexpr (u < 8) {
                            float unused = 0.0f;
                            if (masked_n) head_unit(IC<1 - P>{}, IC<u>{}, n0 + BN, true, unused);
                        }
                    });
                }
            }
            if constexpr (i < DEFER) {  // a deferred exponential unit and its row-sum term
                constexpr int u = 16 - DEFER + i;
                static_assert(DEFER == 0 || QK_SLOTS + (u >> 2) * F::DTILES > i, "P is ready before the P.V slot that multiplies with it");
                exp_unit(IC<u>{});
                lsum = PVT::dot2_ones(pf[u >> 2], u & 3, lsum);
                asm volatile("" ::"v"(lsum));
            }
            __builtin_amdgcn_sched_barrier(0);
        });
        l_i += lsum;
        mslot = mslot_next;
        if (step + 4 < nsteps) { k_fetch += k_tile_bytes; k_tile++; }  // next iteration fetches K of step+4, V of step+3
        if (step + 3 < nsteps) { v_fetch += v_tile_bytes; v_tile++; }
        __builtin_amdgcn_s_setprio(0);
        // (additive mask: the entries of the next step, requested ahead of this step's K/V loads, have landed)
        if constexpr (MF32) __builtin_amdgcn_s_waitcnt(0x0F70);
        else if constexpr (MADD) __builtin_amdgcn_s_waitcnt(0x0F70 | NDMA_KV);
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): every fragment read of this phase has returned
        __builtin_amdgcn_s_barrier();        // phase switch: this wave goes back to the VALU
        __builtin_amdgcn_sched_barrier(0);
    };

    if (wave >= kFastWaves / 2) __syncthreads();  // second half of the waves runs one phase behind
    // The loop always runs an even number of steps (no exit between the two parities: the accumulators
    // then stay in one set of registers); after an odd nsteps the extra step multiplies V by P = 0.
    // Steps before `hide_from` (even) take the lean body: step s hides keys when its tile reaches past the limit
    // of the wave's first row, which the body of step s - 1 prepares; a ragged last tile is fetched three (K) or
    // two (V) steps ahead.
    int hide_from = 0;
    if (CAUSAL) {
        const int first_hidden_step = (__builtin_amdgcn_readfirstlane(wlim) + 1) / BN;  // tile that holds key wlim + 1 (may lie past the last step); wave-uniform
        hide_from = max(min(first_hidden_step - 1, ragged ? nk - 4 : nsteps), 0) & ~1;
    }
    int step = 0;
    if (CAUSAL) {
        for (; step < min(hide_from, nsteps); step += 2) {
            body(IC<0>{}, IC<0>{}, step);
            body(IC<1>{}, IC<0>{}, step + 1);
        }
    }
    for (; step < nsteps; step += 2) {
        body(IC<0>{}, IC<1>{}, step);
        body(IC<1>{}, IC<1>{}, step + 1);
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);  // every direct-to-LDS load of this wave has landed
    if (wave < kFastWaves / 2) __syncthreads();
    __syncthreads();  // nobody reads or fills a K/V tile any more: the LDS is free for the output
    // ---- epilogue: O = O^T / l, lse = log2(l) + m
    // (the instances that take the row sums with v_dot2 hold half a row's sum per lane)
    const float l_o = __shfl_xor(l_i, 32);
    const float l_tot = kWholeRowSums ? l_i : half ? (l_o + l_i) : (l_i + l_o);
    const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;  // l = 0: a row that saw no key; its output is 0, its lse -inf
    const int64_t obase_wave = (int64_t)b * a.os_b + (int64_t)h * a.os_h + (int64_t)(m0 + 32 * wave) * a.os_n + split * a.out_split_stride;
    if (a.out_dt != SAGE_F32) {
        // 16-bit outputs: a lane holds its row in 8-byte pieces, which stored directly would scatter 32
        // partial lines per instruction.  Each wave transposes its 32 rows through its own slice of LDS
        // and writes whole rows, 16 bytes per lane.
        constexpr int ORS = 2 * D + 16;  // bytes per staged row
        static_assert(kFastWaves * 32 * ORS <= F::TOTAL, "output staging fits in the tile buffers");
        unsigned char* mine = smem + wave * 32 * ORS;
#pragma unroll
        for (int dt = 0; dt < F::DTILES; dt++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                float r[4];
#pragma unroll
                for (int i = 0; i < 4; i++) r[i] = o[dt][4 * g + i] * inv;
                s16x4 w;
                if (a.out_dt == SAGE_BF16) {
                    typedef __bf16 b4 __attribute__((ext_vector_type(4)));
                    w = __builtin_bit_cast(s16x4, b4{(__bf16)r[0], (__bf16)r[1], (__bf16)r[2], (__bf16)r[3]});
                } else {
                    typedef _Float16 h4 __attribute__((ext_vector_type(4)));
                    w = __builtin_bit_cast(s16x4, h4{(_Float16)r[0], (_Float16)r[1], (_Float16)r[2], (_Float16)r[3]});
                }
                *reinterpret_cast<s16x4*>(mine + l32 * ORS + 2 * (32 * dt + 8 * g + 4 * half)) = w;
            }
        asm volatile("" ::: "memory");  // the reads below see other lanes' writes (same wave: LDS keeps program order)
        constexpr int LPR = 2 * D / 16, RPI = 64 / LPR;  // lanes per row, rows per wave instruction
        unsigned char* outp = reinterpret_cast<unsigned char*>(a.out) + 2 * obase_wave + 16 * (lane % LPR);
#pragma unroll
        for (int e = 0; e < 32 / RPI; e++) {
            const int r = RPI * e + lane / LPR;
            const v4i piece = *reinterpret_cast<const v4i*>(mine + r * ORS + 16 * (lane % LPR));
            if (m0 + 32 * wave + r < a.M) *reinterpret_cast<v4i*>(outp + 2 * (int64_t)r * a.os_n) = piece;
        }
    } else if (row_ok) {
        float* outp = static_cast<float*>(a.out) + obase_wave + (int64_t)l32 * a.os_n;
#pragma unroll
        for (int dt = 0; dt < F::DTILES; dt++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int d = 32 * dt + 8 * g + 4 * half;
                *reinterpret_cast<v4f*>(outp + d) = v4f{o[dt][4 * g] * inv, o[dt][4 * g + 1] * inv, o[dt][4 * g + 2] * inv, o[dt][4 * g + 3] * inv};
            }
    }
    if (row_ok) {
        if (a.lse && half == 0) a.lse[((int64_t)b * a.Hq + h) * a.M + my_m + split * a.lse_split_stride] = (__builtin_log2f(l_tot) + m_i) * a.lse_mul;
    }
    __syncthreads();  // the output staging in LDS has been read: the next q-block may fill the tile buffers
  }
}

}  // namespace
}  // namespace attn
}  // namespace sage
