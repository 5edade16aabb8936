// Per-block INT8 quantization of Q and K (with the `k - km` smoothing fused in) and the
// fixed-order K mean, for gfx950.
//
// Arithmetic follows quant_per_block_int8_kernel (FlagAttention
// src/flag_attn/sage_attention/quant_per_block.py:38-46) operation by operation in IEEE fp32:
//   x = fp32(in) [* sm_scale];  scale = max|x| / 127;  y = x / scale;  y += (y >= 0 ? .5 : -.5);
//   q = (int8) truncate(y)
// and `k - km` (:53-54) is one fp32 subtraction rounded once to the promoted dtype.
//
// HBM-bound: one workgroup per [BLK, D] block reads the block once (16-byte loads, coalesced
// along head_dim), keeps it in registers as fp32, reduces max|x| with wave shuffles plus one LDS
// step, and writes 8-byte int8 groups.  Algorithmic traffic: in_bytes + 1 byte per element.
#include <mutex>

#include "common.h"

namespace sage {
namespace {

constexpr int kThreads = 256;

// Chunk partials of the K mean for the entry point that takes no workspace (sage_k_mean_noalloc).  Each GPU
// holds its own copy of this array, at its own address, until the process ends; the name below is a host-side
// handle only, so every use goes through the address hipGetSymbolAddress returns for the current device.
constexpr size_t kScratchBytes = SAGE_K_MEAN_NOALLOC_MAX_WORKSPACE_BYTES;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};  // per device: address of that device's copy of `scratch`

struct QuantArgs {
    const void* x;
    const void* km;
    int8_t* out;
    float* scale;
    int64_t xs_b, xs_h, xs_n;
    int64_t ks_b, ks_h, ks_n;
    int64_t os_b, os_h, os_n;
    int32_t H, L, D8, d8_shift, blk, nblk;
    int32_t km_dt, diff_dt;
    int32_t apply_mul;
    float mul;
    // Optional (Q blocks of the K-smoothing entry point): dot[b, h, n] = sum_d fp32(x[b, h, n, d]) * fp32(km[b, h / dot_groups, d]),
    // the per-row shift K smoothing takes out of every logit of row n.  km is then NOT subtracted from x.
    float* dot;
    int32_t dot_groups;
    int32_t small_offsets;  // every byte offset inside one block of x and of out fits 31 bits (host-checked)
};

__device__ __forceinline__ void unpack8(const uint4& r, int dt, float (&v)[8]) {
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
    if (dt == SAGE_BF16) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            v[2 * i] = __builtin_bit_cast(float, w[i] << 16);
            v[2 * i + 1] = __builtin_bit_cast(float, w[i] & 0xffff0000u);
        }
    } else {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            v[2 * i] = (float)__builtin_bit_cast(_Float16, (uint16_t)(w[i] & 0xffffu));
            v[2 * i + 1] = (float)__builtin_bit_cast(_Float16, (uint16_t)(w[i] >> 16));
        }
    }
}

template <int DT>
__device__ __forceinline__ void load8(const void* base, int64_t elem_off, float (&v)[8]) {
    if constexpr (DT == SAGE_F32) {
        const float4* p = reinterpret_cast<const float4*>(static_cast<const float*>(base) + elem_off);
        float4 a = p[0], b = p[1];
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
        v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    } else {
        uint4 r = *reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(base) + elem_off);
        unpack8(r, DT, v);
    }
}

__device__ __forceinline__ void load8_rt(const void* base, int dt, int64_t elem_off, float (&v)[8]) {
    if (dt == SAGE_F32) load8<SAGE_F32>(base, elem_off, v);
    else if (dt == SAGE_BF16) load8<SAGE_BF16>(base, elem_off, v);
    else load8<SAGE_F16>(base, elem_off, v);
}

__device__ __forceinline__ float round_to(float x, int dt) {
    if (dt == SAGE_BF16) return (float)(__bf16)x;
    if (dt == SAGE_F16) return (float)(_Float16)x;
    return x;
}

// Four quantized values -> four bytes of one register (v_perm_b32 picks the low byte of each).
__device__ __forceinline__ uint32_t pack4(int q0, int q1, int q2, int q3) {
    const uint32_t lo = __builtin_amdgcn_perm((uint32_t)q1, (uint32_t)q0, 0x0c0c0400u);
    const uint32_t hi = __builtin_amdgcn_perm((uint32_t)q3, (uint32_t)q2, 0x04000c0cu);
    return lo | hi;
}

// x / scale for the eight values of a unit, then round half away from zero and pack.
// x / scale, correctly rounded, without a division per element: with r = RN(1 / scale) (one IEEE
// division per block), q0 = x * r is within 1.5 ulp of the quotient; one residual correction
// q1 = fma(fma(-q0, scale, x), r, q0) is a faithful rounding, for which the residual is exact, and a
// second one is then the correctly rounded quotient (Markstein's division theorem).  Scales whose
// reciprocal could overflow or whose significand is all ones take the hardware division instead.
__device__ __forceinline__ uint2 quantize8(const float (&v)[8], float scale, float rcp, bool fast_div) {
    float y[8];
    if (fast_div) {
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const float x = v[e];
            const float q0 = x * rcp;
            const float q1 = __builtin_fmaf(__builtin_fmaf(-q0, scale, x), rcp, q0);
            y[e] = __builtin_fmaf(__builtin_fmaf(-q1, scale, x), rcp, q1);
        }
    } else {
#pragma unroll
        for (int e = 0; e < 8; e++) y[e] = v[e] / scale;  // IEEE fp32 divide (hipcc default is correctly rounded)
    }
    int q[8];
#pragma unroll
    for (int e = 0; e < 8; e++) {
        const float t = y[e] + __builtin_copysignf(0.5f, y[e]);  // reference: y + 0.5 * sign(y), sign(0) = +
        q[e] = (int)t;                                           // truncation toward zero; |t| <= 128
    }
    return make_uint2(pack4(q[0], q[1], q[2], q[3]), pack4(q[4], q[5], q[6], q[7]));
}

// max |x| of the workgroup (every thread gets it)
template <int THREADS>
__device__ __forceinline__ float block_amax(float amax, float* wave_max) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off));
    const int tid = threadIdx.x;
    if ((tid & 63) == 0) wave_max[tid >> 6] = amax;
    __syncthreads();
    amax = wave_max[0];
#pragma unroll
    for (int w = 1; w < THREADS / 64; w++) amax = fmaxf(amax, wave_max[w]);
    return amax;
}

// One workgroup = one quantization block of `blk` rows; UNITS 8-element groups per thread.
// wave_max: THREADS / 64 floats of LDS.
template <int DT, int UNITS, int THREADS>
__device__ __forceinline__ void quant_block(const QuantArgs& a, int bid, float* wave_max) {
    const int tid = threadIdx.x;
    const int ib = bid % a.nblk;
    const int h = (bid / a.nblk) % a.H;
    const int b = bid / (a.nblk * a.H);
    const int total_units = a.blk * a.D8;

    const int64_t x_base = (int64_t)b * a.xs_b + (int64_t)h * a.xs_h;
    const int64_t o_base = (int64_t)b * a.os_b + (int64_t)h * a.os_h;
    const int hm = a.dot ? h / a.dot_groups : h;  // head of km (grouped heads when km belongs to K and x is Q)
    const int64_t k_base = (int64_t)b * a.ks_b + (int64_t)hm * a.ks_h;

    // When km is broadcast along the sequence (stride 0) and head_dim / 8 is a power of two not above
    // the thread count, a thread keeps its channel group for all its units, so the K mean of that
    // group is loaded once.
    const bool fixed_c8 = a.ks_n == 0 && a.d8_shift >= 0 && a.D8 <= THREADS;
    float m_fixed[8];
    if (a.km && fixed_c8) load8_rt(a.km, a.km_dt, k_base + (tid & (a.D8 - 1)) * 8, m_fixed);

    constexpr int ESZ = DT == SAGE_F32 ? 4 : 2;
    // ---- The common case, a block that lies whole inside the sequence and fills every unit of every thread:
    //      row and channel group of a thread are fixed, unit j is `rpp` rows further down, so every address is
    //      a uniform base plus one 32-bit per-thread offset, nothing is masked and nothing is clamped.
    const bool whole = a.d8_shift >= 0 && a.D8 <= THREADS && total_units == UNITS * THREADS && (ib + 1) * a.blk <= a.L &&
                       (!a.km || fixed_c8) && a.small_offsets;
    if (whole) {
        const int row0 = tid >> a.d8_shift, c8 = tid & (a.D8 - 1);
        const int rpp = THREADS >> a.d8_shift;  // rows per pass of the threads
        const unsigned char* src = static_cast<const unsigned char*>(a.x) + (x_base + (int64_t)ib * a.blk * a.xs_n) * ESZ;
        const uint32_t voff = (uint32_t)((row0 * (int)a.xs_n + c8 * 8) * ESZ);
        const int64_t pass_bytes = (int64_t)rpp * a.xs_n * ESZ;
        uint4 raw16[UNITS];
        float4 raw32[UNITS][2];
#pragma unroll
        for (int j = 0; j < UNITS; j++) {
            const unsigned char* p = src + j * pass_bytes + voff;
            if constexpr (DT == SAGE_F32) {
                raw32[j][0] = reinterpret_cast<const float4*>(p)[0];
                raw32[j][1] = reinterpret_cast<const float4*>(p)[1];
            } else {
                raw16[j] = *reinterpret_cast<const uint4*>(p);
            }
        }
        float v[UNITS][8];
        float amax = 0.0f;
#pragma unroll
        for (int j = 0; j < UNITS; j++) {
            if constexpr (DT == SAGE_F32) {
                v[j][0] = raw32[j][0].x; v[j][1] = raw32[j][0].y; v[j][2] = raw32[j][0].z; v[j][3] = raw32[j][0].w;
                v[j][4] = raw32[j][1].x; v[j][5] = raw32[j][1].y; v[j][6] = raw32[j][1].z; v[j][7] = raw32[j][1].w;
            } else {
                unpack8(raw16[j], DT, v[j]);
            }
            if (a.dot) {
                // dot of the row with km: eight terms in order per thread, then the D8 threads of the row pairwise
                float d = 0.0f;
#pragma unroll
                for (int e = 0; e < 8; e++) d = d + v[j][e] * m_fixed[e];
                for (int off = 1; off < a.D8; off <<= 1) d = d + __shfl_xor(d, off);
                if (c8 == 0) a.dot[((int64_t)b * a.H + h) * a.L + ib * a.blk + row0 + j * rpp] = d;
            } else if (a.km) {
#pragma unroll
                for (int e = 0; e < 8; e++) v[j][e] = round_to(v[j][e] - m_fixed[e], a.diff_dt);
            }
            if (a.apply_mul) {
#pragma unroll
                for (int e = 0; e < 8; e++) v[j][e] = v[j][e] * a.mul;
            }
#pragma unroll
            for (int e = 0; e < 8; e += 2) amax = fmaxf(fmaxf(amax, fabsf(v[j][e])), fabsf(v[j][e + 1]));
        }
        amax = block_amax<THREADS>(amax, wave_max);
        const float scale = amax / 127.0f;
        if (tid == 0) a.scale[((int64_t)b * a.H + h) * a.nblk + ib] = scale;
        const bool zero_block = !(scale > 0.0f);  // 0/0 -> NaN in the reference; its int8 conversion yields 0
        const uint32_t sbits = __builtin_bit_cast(uint32_t, scale);
        const bool fast_div = scale >= 0x1p-60f && scale <= 0x1p60f && (sbits & 0x7fffffu) != 0x7fffffu;
        const float rcp = 1.0f / scale;
        unsigned char* dst = reinterpret_cast<unsigned char*>(a.out) + o_base + (int64_t)ib * a.blk * a.os_n;
        const uint32_t ooff = (uint32_t)(row0 * (int)a.os_n + c8 * 8);
        const int64_t opass = (int64_t)rpp * a.os_n;
#pragma unroll
        for (int j = 0; j < UNITS; j++) {
            const uint2 packed = zero_block ? make_uint2(0u, 0u) : quantize8(v[j], scale, rcp, fast_div);
            *reinterpret_cast<uint2*>(dst + j * opass + ooff) = packed;
        }
        return;
    }

    // ---- any other block (tail of the sequence, odd block sizes, km that varies along the sequence).
    // All loads of the block are issued before anything waits for one: they are unconditional (a unit
    // past the end of the block or of the sequence re-reads a valid row and is zeroed afterwards), so
    // that the compiler keeps them together instead of one load, one wait per unit.
    uint4 raw16[UNITS];
    float4 raw32[UNITS][2];
    bool live[UNITS];
    int64_t koff[UNITS];  // km entry of the unit when km is not one row per (batch, head) (loaded where it is used)
#pragma unroll
    for (int j = 0; j < UNITS; j++) {
        const int u = min(tid + THREADS * j, total_units - 1);
        int row, c8;
        if (a.d8_shift >= 0) {
            row = u >> a.d8_shift;
            c8 = u & (a.D8 - 1);
        } else {
            row = u / a.D8;
            c8 = u - row * a.D8;
        }
        const int n = ib * a.blk + row;
        live[j] = (tid + THREADS * j < total_units) && (n < a.L);
        const int64_t nc = min(n, a.L - 1);
        const int64_t off = x_base + nc * a.xs_n + c8 * 8;
        if constexpr (DT == SAGE_F32) {
            const float4* p = reinterpret_cast<const float4*>(static_cast<const float*>(a.x) + off);
            raw32[j][0] = p[0];
            raw32[j][1] = p[1];
        } else {
            raw16[j] = *reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(a.x) + off);
        }
        koff[j] = k_base + nc * a.ks_n + c8 * 8;
    }

    float v[UNITS][8];
    float amax = 0.0f;
#pragma unroll
    for (int j = 0; j < UNITS; j++) {
        if constexpr (DT == SAGE_F32) {
            v[j][0] = raw32[j][0].x; v[j][1] = raw32[j][0].y; v[j][2] = raw32[j][0].z; v[j][3] = raw32[j][0].w;
            v[j][4] = raw32[j][1].x; v[j][5] = raw32[j][1].y; v[j][6] = raw32[j][1].z; v[j][7] = raw32[j][1].w;
        } else {
            unpack8(raw16[j], DT, v[j]);
        }
        if (a.km) {
            float m[8];
            if (fixed_c8) {
#pragma unroll
                for (int e = 0; e < 8; e++) m[e] = m_fixed[e];
            } else {
                load8_rt(a.km, a.km_dt, koff[j], m);
            }
            if (a.dot) {
                // (the entry point that asks for the dot passes a km of one row per head and a power-of-two
                // head_dim / 8 <= 64: the threads of a row are then neighbours inside one wave)
                float d = 0.0f;
#pragma unroll
                for (int e = 0; e < 8; e++) d = d + v[j][e] * m[e];
                for (int off = 1; off < a.D8; off <<= 1) d = d + __shfl_xor(d, off);
                const int u = tid + THREADS * j;
                const int row = u >> a.d8_shift;
                if (live[j] && (u & (a.D8 - 1)) == 0) a.dot[((int64_t)b * a.H + h) * a.L + ib * a.blk + row] = d;
            } else {
#pragma unroll
                for (int e = 0; e < 8; e++) v[j][e] = round_to(v[j][e] - m[e], a.diff_dt);
            }
        }
        if (a.apply_mul) {
#pragma unroll
            for (int e = 0; e < 8; e++) v[j][e] = v[j][e] * a.mul;
        }
        if (!live[j]) {
#pragma unroll
            for (int e = 0; e < 8; e++) v[j][e] = 0.0f;  // rows past L are masked loads: zeros
        }
#pragma unroll
        for (int e = 0; e < 8; e++) amax = fmaxf(amax, fabsf(v[j][e]));
    }

    amax = block_amax<THREADS>(amax, wave_max);
    const float scale = amax / 127.0f;
    if (tid == 0) a.scale[((int64_t)b * a.H + h) * a.nblk + ib] = scale;
    const bool zero_block = !(scale > 0.0f);  // 0/0 -> NaN in the reference; its int8 conversion yields 0
    const uint32_t sbits = __builtin_bit_cast(uint32_t, scale);
    const bool fast_div = scale >= 0x1p-60f && scale <= 0x1p60f && (sbits & 0x7fffffu) != 0x7fffffu;
    const float rcp = 1.0f / scale;

#pragma unroll
    for (int j = 0; j < UNITS; j++) {
        const int u = tid + THREADS * j;
        int row, c8;
        if (a.d8_shift >= 0) {
            row = u >> a.d8_shift;
            c8 = u & (a.D8 - 1);
        } else {
            row = u / a.D8;
            c8 = u - row * a.D8;
        }
        const int n = ib * a.blk + row;
        if (live[j]) {
            const uint2 packed = zero_block ? make_uint2(0u, 0u) : quantize8(v[j], scale, rcp, fast_div);
            *reinterpret_cast<uint2*>(a.out + o_base + (int64_t)n * a.os_n + c8 * 8) = packed;
        }
    }
}

template <int DT, int UNITS, int THREADS>
__global__ __launch_bounds__(THREADS) void quant_per_block_int8_kernel(QuantArgs a) {
    __shared__ float wave_max[THREADS / 64];
    quant_block<DT, UNITS, THREADS>(a, blockIdx.x, wave_max);
}

template <int DT>
int launch_one(const QuantArgs& a, int64_t nblocks, hipStream_t stream) {
    // four 16-byte loads in flight per thread wherever the block is large enough, and a register
    // footprint that keeps eight waves per SIMD resident
    const int total_units = a.blk * a.D8;
    dim3 grid((unsigned)nblocks);
    if (total_units <= 256) hipLaunchKernelGGL((quant_per_block_int8_kernel<DT, 1, 256>), grid, dim3(256), 0, stream, a);
    else if (total_units <= 512) hipLaunchKernelGGL((quant_per_block_int8_kernel<DT, 2, 256>), grid, dim3(256), 0, stream, a);
    else if (total_units <= 1024) hipLaunchKernelGGL((quant_per_block_int8_kernel<DT, 4, 256>), grid, dim3(256), 0, stream, a);
    else if (total_units <= 2048) hipLaunchKernelGGL((quant_per_block_int8_kernel<DT, 4, 512>), grid, dim3(512), 0, stream, a);
    else hipLaunchKernelGGL((quant_per_block_int8_kernel<DT, 8, 512>), grid, dim3(512), 0, stream, a);
    return check_launch("quant_per_block_int8_kernel");
}

int launch_tensor(const QuantArgs& a, int in_dtype, int64_t nblocks, hipStream_t stream) {
    if (nblocks <= 0) return SAGE_OK;
    if (nblocks > 0x7fffffffLL) return fail(SAGE_E_UNSUPPORTED, "sage_per_block_int8: too many blocks");
    switch (in_dtype) {
        case SAGE_F16: return launch_one<SAGE_F16>(a, nblocks, stream);
        case SAGE_BF16: return launch_one<SAGE_BF16>(a, nblocks, stream);
        default: return launch_one<SAGE_F32>(a, nblocks, stream);
    }
}

bool aligned_to(int align, const void* p, int esz, int64_t s0, int64_t s1, int64_t s2) {
    return ((uintptr_t)p % align) == 0 && (s0 * esz) % align == 0 && (s1 * esz) % align == 0 &&
           (s2 * esz) % align == 0;
}
bool aligned16(const void* p, int esz, int64_t s0, int64_t s1, int64_t s2) {
    return aligned_to(16, p, esz, s0, s1, s2);
}

// ---------------------------------------------------------------------------------------------
// K mean, fixed order.  Stage 1: one thread per (chunk of 64 rows, 4 channels) adds the rows in
// order.  Stage 2: one thread per channel adds the chunk partials in order, divides, rounds.
// ---------------------------------------------------------------------------------------------
struct KMeanArgs {
    const void* k;
    float* part;  // [B*H, nchunk, D]
    void* out;    // [B*H, D]
    int64_t s_b, s_h, s_n;
    int32_t H, N, D, D8, nchunk, out_dt;
    int64_t total_items;  // B*H*nchunk*D8
};

// W consecutive channels of one row as fp32 (W = 8, 4 or 2; 16-bit inputs load 2 * W bytes)
template <int DT, int W>
__device__ __forceinline__ void loadw(const void* base, int64_t elem_off, float (&v)[W]) {
    if constexpr (W == 8) {
        load8<DT>(base, elem_off, v);
    } else if constexpr (DT == SAGE_F32) {
        const float* p = static_cast<const float*>(base) + elem_off;
        if constexpr (W == 4) {
            const float4 r = *reinterpret_cast<const float4*>(p);
            v[0] = r.x; v[1] = r.y; v[2] = r.z; v[3] = r.w;
        } else {
            const float2 r = *reinterpret_cast<const float2*>(p);
            v[0] = r.x; v[1] = r.y;
        }
    } else {
        const uint16_t* p = static_cast<const uint16_t*>(base) + elem_off;
        uint32_t w[W / 2];
        if constexpr (W == 4) {
            const uint2 r = *reinterpret_cast<const uint2*>(p);
            w[0] = r.x; w[1] = r.y;
        } else {
            w[0] = *reinterpret_cast<const uint32_t*>(p);
        }
#pragma unroll
        for (int i = 0; i < W / 2; i++) {
            if constexpr (DT == SAGE_BF16) {
                v[2 * i] = __builtin_bit_cast(float, w[i] << 16);
                v[2 * i + 1] = __builtin_bit_cast(float, w[i] & 0xffff0000u);
            } else {
                v[2 * i] = (float)__builtin_bit_cast(_Float16, (uint16_t)(w[i] & 0xffffu));
                v[2 * i + 1] = (float)__builtin_bit_cast(_Float16, (uint16_t)(w[i] >> 16));
            }
        }
    }
}

// One thread per (chunk of 64 rows, W channels): narrow W means more threads in flight for the same
// bytes; a wave still reads whole contiguous row segments (64 * W elements).
template <int DT, int W>
__device__ __forceinline__ void k_mean_partial_item(const KMeanArgs& a, int64_t item) {
    if (item >= a.total_items) return;
    const int dw = a.D / W;
    const int cw = (int)(item % dw);
    const int64_t t = item / dw;
    const int chunk = (int)(t % a.nchunk);
    const int64_t bh = t / a.nchunk;
    const int h = (int)(bh % a.H);
    const int64_t b = bh / a.H;
    const int64_t base = b * a.s_b + (int64_t)h * a.s_h + cw * W;
    float acc[W];
#pragma unroll
    for (int e = 0; e < W; e++) acc[e] = 0.0f;
    const int n0 = chunk * 64;
    const int rows = min(64, a.N - n0);
    int r = 0;
    constexpr int kBatch = 16;  // rows whose loads are in flight together
    for (; r + kBatch <= rows; r += kBatch) {
        float v[kBatch][W];
#pragma unroll
        for (int i = 0; i < kBatch; i++) loadw<DT, W>(a.k, base + (int64_t)(n0 + r + i) * a.s_n, v[i]);
#pragma unroll
        for (int i = 0; i < kBatch; i++)
#pragma unroll
            for (int e = 0; e < W; e++) acc[e] = acc[e] + v[i][e];
    }
    for (; r < rows; r++) {
        float v[W];
        loadw<DT, W>(a.k, base + (int64_t)(n0 + r) * a.s_n, v);
#pragma unroll
        for (int e = 0; e < W; e++) acc[e] = acc[e] + v[e];
    }
    float* dst = a.part + (bh * a.nchunk + chunk) * a.D + cw * W;
#pragma unroll
    for (int e = 0; e < W; e++) dst[e] = acc[e];
}

template <int DT, int W>
__global__ __launch_bounds__(kThreads) void k_mean_partial_kernel(KMeanArgs a) {
    k_mean_partial_item<DT, W>(a, (int64_t)blockIdx.x * kThreads + threadIdx.x);
}

// First launch of the K-smoothing entry point: the Q quantization blocks and the chunk partials of the K mean
// do not depend on each other, so they share one grid (the quantizer is bound by its arithmetic, the partial
// sums by memory latency: side by side they take less than one after the other).  Workgroup i serves the K mean
// when i is a multiple of `period` (and partial blocks are left), a Q block otherwise.
constexpr int kStage1Threads = 512;
constexpr int kMeanW = 4;  // channels per thread of the partial sums: 8-byte loads of 16-bit inputs, twice the threads of 16-byte loads
template <int DT, int UNITS>
__global__ __launch_bounds__(kStage1Threads) void smooth_stage1_kernel(QuantArgs qa, KMeanArgs ka, int n_partial, int period) {
    __shared__ float wave_max[kStage1Threads / 64];
    const int i = blockIdx.x;
    const int before = min(n_partial, (i + period - 1) / period);  // K-mean workgroups among 0 .. i-1
    if (i % period == 0 && i / period < n_partial) {
        k_mean_partial_item<DT, kMeanW>(ka, (int64_t)(i / period) * kStage1Threads + threadIdx.x);
    } else {
        quant_block<DT, UNITS, kStage1Threads>(qa, i - before, wave_max);
    }
}

__global__ __launch_bounds__(kThreads) void k_mean_final_kernel(KMeanArgs a, int64_t channels) {
    const int64_t ch = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;  // (b*H + h) * D + d
    if (ch >= channels) return;
    const int64_t bh = ch / a.D;
    const int d = (int)(ch % a.D);
    const float* p = a.part + bh * a.nchunk * a.D + d;
    float tot = 0.0f;
    int c = 0;
    for (; c + 32 <= a.nchunk; c += 32) {  // loads issued together, additions kept in chunk order
        float v[32];
#pragma unroll
        for (int i = 0; i < 32; i++) v[i] = p[(int64_t)(c + i) * a.D];
#pragma unroll
        for (int i = 0; i < 32; i++) tot = tot + v[i];
    }
    for (; c + 8 <= a.nchunk; c += 8) {
        float v[8];
#pragma unroll
        for (int i = 0; i < 8; i++) v[i] = p[(int64_t)(c + i) * a.D];
#pragma unroll
        for (int i = 0; i < 8; i++) tot = tot + v[i];
    }
    for (; c < a.nchunk; c++) tot = tot + p[(int64_t)c * a.D];
    const float mean = tot / (float)a.N;
    if (a.out_dt == SAGE_F32) static_cast<float*>(a.out)[ch] = mean;
    else if (a.out_dt == SAGE_BF16) static_cast<__bf16*>(a.out)[ch] = (__bf16)mean;
    else static_cast<_Float16*>(a.out)[ch] = (_Float16)mean;
}

}  // namespace

// Address of the current device's copy of the static scratch array (looked up once per device).
int static_scratch(void** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(SAGE_E_LAUNCH, "hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= kMaxDevices) return fail(SAGE_E_UNSUPPORTED, "device index %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr)
            return fail(SAGE_E_LAUNCH, "hipGetSymbolAddress(scratch) on device %d: %s", dev, hipGetErrorString(e));
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return SAGE_OK;
}

namespace {

int d8_shift_of(int64_t D) {
    const int D8 = (int)(D / 8);
    if ((D8 & (D8 - 1)) != 0) return -1;
    int shift = 0;
    while ((1 << shift) < D8) shift++;
    return shift;
}

bool fits31(int64_t rows, int64_t stride, int esz) { return stride >= 0 && rows * stride * esz < (1LL << 31); }

// Arguments of the K launch (with_km: subtract p.km) / of the Q launch.  Returns a status.
int k_args(const sage_quant_params& p, bool with_km, QuantArgs& a) {
    const int esz = dtype_bytes(p.in_dtype);
    if (!aligned16(p.k.ptr, esz, p.k.stride_b, p.k.stride_h, p.k.stride_n) ||
        !aligned_to(8, p.k_int8.ptr, 1, p.k_int8.stride_b, p.k_int8.stride_h, p.k_int8.stride_n))
        return fail(SAGE_E_INVALID, "sage_per_block_int8: k rows must be 16-byte aligned (8-byte for int8 output)");
    a = QuantArgs{};
    a.x = p.k.ptr; a.out = (int8_t*)p.k_int8.ptr; a.scale = p.k_scale;
    a.xs_b = p.k.stride_b; a.xs_h = p.k.stride_h; a.xs_n = p.k.stride_n;
    a.os_b = p.k_int8.stride_b; a.os_h = p.k_int8.stride_h; a.os_n = p.k_int8.stride_n;
    if (with_km && p.km.ptr) {
        if (!aligned16(p.km.ptr, dtype_bytes(p.km_dtype), p.km.stride_b, p.km.stride_h, p.km.stride_n))
            return fail(SAGE_E_INVALID, "sage_per_block_int8: km rows must be 16-byte aligned");
        a.km = p.km.ptr; a.ks_b = p.km.stride_b; a.ks_h = p.km.stride_h; a.ks_n = p.km.stride_n;
        a.km_dt = p.km_dtype; a.diff_dt = p.diff_dtype;
    }
    a.H = (int)p.heads_kv; a.L = (int)p.kv_len; a.D8 = (int)(p.head_dim / 8); a.d8_shift = d8_shift_of(p.head_dim); a.blk = p.blkk;
    a.nblk = (int)((p.kv_len + p.blkk - 1) / p.blkk);
    a.apply_mul = 0; a.mul = 1.0f;
    a.small_offsets = fits31(p.blkk, p.k.stride_n, esz) && fits31(p.blkk, p.k_int8.stride_n, 1);
    return SAGE_OK;
}

int q_args(const sage_quant_params& p, QuantArgs& a) {
    const int esz = dtype_bytes(p.in_dtype);
    if (!aligned16(p.q.ptr, esz, p.q.stride_b, p.q.stride_h, p.q.stride_n) ||
        !aligned_to(8, p.q_int8.ptr, 1, p.q_int8.stride_b, p.q_int8.stride_h, p.q_int8.stride_n))
        return fail(SAGE_E_INVALID, "sage_per_block_int8: q rows must be 16-byte aligned (8-byte for int8 output)");
    a = QuantArgs{};
    a.x = p.q.ptr; a.km = nullptr; a.out = (int8_t*)p.q_int8.ptr; a.scale = p.q_scale;
    a.xs_b = p.q.stride_b; a.xs_h = p.q.stride_h; a.xs_n = p.q.stride_n;
    a.os_b = p.q_int8.stride_b; a.os_h = p.q_int8.stride_h; a.os_n = p.q_int8.stride_n;
    a.H = (int)p.heads_q; a.L = (int)p.qo_len; a.D8 = (int)(p.head_dim / 8); a.d8_shift = d8_shift_of(p.head_dim); a.blk = p.blkq;
    a.nblk = (int)((p.qo_len + p.blkq - 1) / p.blkq);
    a.apply_mul = (p.q_mul != 1.0f); a.mul = p.q_mul;
    a.small_offsets = fits31(p.blkq, p.q.stride_n, esz) && fits31(p.blkq, p.q_int8.stride_n, 1);
    return SAGE_OK;
}

int k_mean_args(const sage_tensor& k, int k_dtype, void* km_out, int out_dtype, int64_t B, int64_t H, int64_t N, int64_t D,
                void* workspace, KMeanArgs& a) {
    if (D % 8 != 0) return fail(SAGE_E_UNSUPPORTED, "sage_k_mean: head_dim must be a multiple of 8");
    if (!aligned16(k.ptr, dtype_bytes(k_dtype), k.stride_b, k.stride_h, k.stride_n) || ((uintptr_t)workspace % 16))
        return fail(SAGE_E_INVALID, "sage_k_mean: k rows and workspace must be 16-byte aligned");
    a = KMeanArgs{};
    a.k = k.ptr; a.part = (float*)workspace; a.out = km_out;
    a.s_b = k.stride_b; a.s_h = k.stride_h; a.s_n = k.stride_n;
    a.H = (int)H; a.N = (int)N; a.D = (int)D; a.D8 = (int)(D / 8); a.nchunk = (int)((N + 63) / 64);
    a.out_dt = out_dtype;
    a.total_items = B * H * a.nchunk * (D / kMeanW);
    if ((a.total_items + kThreads - 1) / kThreads > 0x7fffffffLL) return fail(SAGE_E_UNSUPPORTED, "sage_k_mean: too many chunks");
    return SAGE_OK;
}

int launch_k_mean_final(const KMeanArgs& a, int64_t channels, hipStream_t stream) {
    constexpr int kFinalThreads = 64;  // few channels (B * H * D): one wave per workgroup spreads them over the CUs
    const int64_t g2 = (channels + kFinalThreads - 1) / kFinalThreads;
    hipLaunchKernelGGL(k_mean_final_kernel, dim3((unsigned)g2), dim3(kFinalThreads), 0, stream, a, channels);
    return check_launch("k_mean_final_kernel");
}

template <int DT>
int launch_stage1(const QuantArgs& qa, const KMeanArgs& ka, int64_t q_blocks, hipStream_t stream, bool& done) {
    const int64_t n_partial = (ka.total_items + kStage1Threads - 1) / kStage1Threads;
    const int64_t total = q_blocks + n_partial;
    const int units = qa.blk * qa.D8;
    done = false;
    if (total > 0x7fffffffLL || n_partial <= 0 || q_blocks <= 0) return SAGE_OK;
    if (units != 2 * kStage1Threads && units != 4 * kStage1Threads) return SAGE_OK;  // other block shapes: separate launches
    const int period = (int)(total / n_partial);
    dim3 grid((unsigned)total), block(kStage1Threads);
    if (units == 4 * kStage1Threads)
        hipLaunchKernelGGL((smooth_stage1_kernel<DT, 4>), grid, block, 0, stream, qa, ka, (int)n_partial, period);
    else
        hipLaunchKernelGGL((smooth_stage1_kernel<DT, 2>), grid, block, 0, stream, qa, ka, (int)n_partial, period);
    done = true;
    return check_launch("smooth_stage1_kernel");
}

int launch_k_mean_partial(const KMeanArgs& a, int k_dtype, hipStream_t stream) {
    const int64_t g1 = (a.total_items + kThreads - 1) / kThreads;
    dim3 block(kThreads);
    switch (k_dtype) {
        case SAGE_F16: hipLaunchKernelGGL((k_mean_partial_kernel<SAGE_F16, kMeanW>), dim3((unsigned)g1), block, 0, stream, a); break;
        case SAGE_BF16: hipLaunchKernelGGL((k_mean_partial_kernel<SAGE_BF16, kMeanW>), dim3((unsigned)g1), block, 0, stream, a); break;
        default: hipLaunchKernelGGL((k_mean_partial_kernel<SAGE_F32, kMeanW>), dim3((unsigned)g1), block, 0, stream, a); break;
    }
    return check_launch("k_mean_partial_kernel");
}

}  // namespace

int launch_quant(const sage_quant_params& p, hipStream_t stream) {
    // K first: a caller that has just taken the K mean finds K still in the memory-side cache.
    if (p.k.ptr && p.kv_len > 0) {
        QuantArgs a;
        if (int rc = k_args(p, true, a)) return rc;
        if (int rc = launch_tensor(a, p.in_dtype, p.batch * p.heads_kv * a.nblk, stream)) return rc;
    }
    if (p.q.ptr && p.qo_len > 0) {
        QuantArgs a;
        if (int rc = q_args(p, a)) return rc;
        if (int rc = launch_tensor(a, p.in_dtype, p.batch * p.heads_q * a.nblk, stream)) return rc;
    }
    return SAGE_OK;
}

int launch_kmean(const sage_tensor& k, int k_dtype, void* km_out, int out_dtype, int64_t B, int64_t H, int64_t N,
                 int64_t D, void* workspace, hipStream_t stream) {
    KMeanArgs a;
    if (int rc = k_mean_args(k, k_dtype, km_out, out_dtype, B, H, N, D, workspace, a)) return rc;
    if (int rc = launch_k_mean_partial(a, k_dtype, stream)) return rc;
    return launch_k_mean_final(a, B * H * D, stream);
}

// K mean -> k - km -> quantization of K, and quantization of Q, in three launches:
//   1. Q blocks and the chunk partials of the K mean, side by side in one grid;
//   2. the mean per channel (chunk partials added in order, one division, one rounding to K's dtype);
//   3. K blocks, subtracting the mean just written.
// With q_dot_km the Q blocks need the mean as well and move behind it: partials, mean, K blocks, Q blocks.
int launch_smooth_quant(const sage_quant_params& p, void* km_out, float* q_dot_km, void* workspace, hipStream_t stream) {
    const int64_t B = p.batch, H = p.heads_kv, N = p.kv_len, D = p.head_dim;
    KMeanArgs ka;
    if (int rc = k_mean_args(p.k, p.in_dtype, km_out, p.in_dtype, B, H, N, D, workspace, ka)) return rc;
    sage_quant_params pk = p;  // the K launch subtracts the mean written by the second launch
    pk.km.ptr = km_out; pk.km.stride_b = H * D; pk.km.stride_h = D; pk.km.stride_n = 0;
    pk.km_dtype = pk.diff_dtype = p.in_dtype;
    QuantArgs kq, qq;
    if (int rc = k_args(pk, true, kq)) return rc;
    const bool have_q = p.q.ptr && p.qo_len > 0;
    if (have_q) {
        if (int rc = q_args(p, qq)) return rc;
    }
    const int64_t q_blocks = have_q ? p.batch * p.heads_q * qq.nblk : 0;
    bool fused = false;
    if (have_q && !q_dot_km) {
        int rc;
        switch (p.in_dtype) {
            case SAGE_F16: rc = launch_stage1<SAGE_F16>(qq, ka, q_blocks, stream, fused); break;
            case SAGE_BF16: rc = launch_stage1<SAGE_BF16>(qq, ka, q_blocks, stream, fused); break;
            default: rc = launch_stage1<SAGE_F32>(qq, ka, q_blocks, stream, fused); break;
        }
        if (rc) return rc;
    }
    if (!fused) {
        if (int rc = launch_k_mean_partial(ka, p.in_dtype, stream)) return rc;
    }
    if (int rc = launch_k_mean_final(ka, B * H * D, stream)) return rc;
    if (int rc = launch_tensor(kq, p.in_dtype, B * H * kq.nblk, stream)) return rc;
    if (have_q && !fused) {
        if (q_dot_km) {
            qq.km = km_out; qq.ks_b = H * D; qq.ks_h = D; qq.ks_n = 0; qq.km_dt = p.in_dtype; qq.diff_dt = p.in_dtype;
            qq.dot = q_dot_km; qq.dot_groups = (int)(p.heads_q / p.heads_kv);
        }
        if (int rc = launch_tensor(qq, p.in_dtype, q_blocks, stream)) return rc;
    }
    return SAGE_OK;
}

}  // namespace sage
