/*
 * Plain-C restatement of FlagAttention's SageAttention path.  TEST INFRASTRUCTURE ONLY:
 * linked by tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg, never by the
 * shipped library.  Build: `make -C oracle` (gcc -O2 -ffp-contract=off, IEEE fp32 throughout).
 *
 * Reference lines followed (paths relative to the FlagAttention checkout):
 *   sage_oracle_quant  src/flag_attn/sage_attention/quant_per_block.py:38-46 (kernel), :53-54 (k - km)
 *   sage_oracle_attn   src/flag_attn/sage_attention/attn_qk_int8_per_block.py:20-72 (KV loop),
 *                      :88-127 (prologue / epilogue / LSE)
 *   sage_oracle_kmean  no reference counterpart (the caller supplies km there); fixed-order
 *                      fp32 mean that defines this build's smooth_k=True
 *
 * Pinned by: tests/test_oracle_pins.py (golden vectors written from the reference kernel under
 * Triton's CPU interpreter; closed forms; agreement with the independent numpy restatement).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

enum { DT_F16 = 0, DT_BF16 = 1, DT_F32 = 2 };

static float bits_to_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static uint32_t f32_to_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

static float bf16_to_f32(uint16_t h) { return bits_to_f32((uint32_t)h << 16); }

static uint16_t f32_to_bf16(float f) { /* round to nearest even, NaN kept quiet */
    uint32_t u = f32_to_bits(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

static float f16_to_f32(uint16_t h) {
    uint32_t s = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 0x1f, m = h & 0x3ff;
    if (e == 0) {
        if (m == 0) return bits_to_f32(s);
        float v = (float)m * (1.0f / 16777216.0f); /* m * 2^-24, exact */
        return (s ? -v : v);
    }
    if (e == 31) return bits_to_f32(s | 0x7f800000u | (m << 13));
    return bits_to_f32(s | ((e + 112) << 23) | (m << 13));
}

static uint16_t f32_to_f16(float f) { /* round to nearest even */
    uint32_t u = f32_to_bits(f), s = (u >> 16) & 0x8000u, a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint16_t)(s | 0x7e00);
    if (a >= 0x477ff000u) return (uint16_t)(s | 0x7c00); /* >= 65520 rounds to inf */
    if (a < 0x38800000u) { /* below 2^-14: subnormal half; a*2^24 rounds (nearest even) to the integer mantissa */
        float v = bits_to_f32(a) * 16777216.0f;
        return (uint16_t)(s | (uint32_t)lrintf(v)); /* v <= 1024; 1024 == smallest normal encoding */
    }
    uint32_t r = a + 0xfffu + ((a >> 13) & 1u);
    return (uint16_t)(s | ((r - 0x38000000u) >> 13));
}

static float load_elem(const void* p, int dt, int64_t i) {
    switch (dt) {
        case DT_F16: return f16_to_f32(((const uint16_t*)p)[i]);
        case DT_BF16: return bf16_to_f32(((const uint16_t*)p)[i]);
        default: return ((const float*)p)[i];
    }
}

static float round_to(float x, int dt) {
    switch (dt) {
        case DT_F16: return f16_to_f32(f32_to_f16(x));
        case DT_BF16: return bf16_to_f32(f32_to_bf16(x));
        default: return x;
    }
}

/*
 * Per-block INT8 quantization of one tensor viewed as [B,H,L,D] through strides (elements,
 * last dim contiguous).  km (may be NULL) is broadcast through its own strides; the
 * difference is rounded once to diff_dtype as torch's `k - km` does (:53-54).
 * apply_mul = 0 reproduces the K call, where sm_scale == 1.0 multiplies nothing.
 */
int sage_oracle_quant(const void* x, int x_dtype, const void* km, int km_dtype, int diff_dtype,
                      int8_t* out, float* scale, int64_t B, int64_t H, int64_t L, int64_t D,
                      int64_t xs_b, int64_t xs_h, int64_t xs_n, int64_t ks_b, int64_t ks_h, int64_t ks_n,
                      int64_t os_b, int64_t os_h, int64_t os_n, int blk, float scale_mul, int apply_mul) {
    int64_t nb = (L + blk - 1) / blk;
    float* tile = (float*)malloc(sizeof(float) * (size_t)blk * (size_t)D);
    if (!tile) return -1;
    for (int64_t b = 0; b < B; b++)
        for (int64_t h = 0; h < H; h++)
            for (int64_t ib = 0; ib < nb; ib++) {
                int64_t rows = L - ib * blk < blk ? L - ib * blk : blk;
                float amax = 0.0f; /* rows past L are masked loads, i.e. zeros (:38) */
                for (int64_t r = 0; r < rows; r++)
                    for (int64_t d = 0; d < D; d++) {
                        int64_t n = ib * blk + r;
                        float v = load_elem(x, x_dtype, b * xs_b + h * xs_h + n * xs_n + d);
                        if (km) {
                            float m = load_elem(km, km_dtype, b * ks_b + h * ks_h + n * ks_n + d);
                            v = round_to(v - m, diff_dtype);
                        }
                        if (apply_mul) v = v * scale_mul; /* :40 */
                        tile[r * D + d] = v;
                        float a = fabsf(v);
                        if (a > amax) amax = a;
                    }
                float sc = amax / 127.0f; /* :41 */
                scale[(b * H + h) * nb + ib] = sc;
                for (int64_t r = 0; r < rows; r++)
                    for (int64_t d = 0; d < D; d++) {
                        float y = tile[r * D + d] / sc;          /* :42 */
                        y = y + (y >= 0.0f ? 0.5f : -0.5f);        /* :43 */
                        int8_t q = 0;
                        if (y == y) {                              /* NaN (0/0 in an all-zero block) -> 0 */
                            float t = truncf(y);                   /* :44 fp -> int truncates toward zero */
                            if (t > 127.0f) t = 127.0f;
                            if (t < -128.0f) t = -128.0f;
                            q = (int8_t)t;
                        }
                        out[b * os_b + h * os_h + (ib * blk + r) * os_n + d] = q;
                    }
            }
    free(tile);
    return 0;
}

/*
 * Fixed-order fp32 mean of K over the sequence axis: rows of each 64-row chunk are added in
 * order from 0.0f, chunk partials are added in order from 0.0f, the total is divided by
 * (float)N and rounded once to out_dtype.  out is [B,H,D] contiguous, written as raw bits.
 */
int sage_oracle_kmean(const void* k, int k_dtype, void* out, int out_dtype, int64_t B, int64_t H, int64_t N,
                      int64_t D, int64_t s_b, int64_t s_h, int64_t s_n) {
    for (int64_t b = 0; b < B; b++)
        for (int64_t h = 0; h < H; h++)
            for (int64_t d = 0; d < D; d++) {
                float tot = 0.0f;
                for (int64_t c = 0; c < N; c += 64) {
                    float part = 0.0f;
                    for (int64_t n = c; n < c + 64 && n < N; n++)
                        part = part + load_elem(k, k_dtype, b * s_b + h * s_h + n * s_n + d);
                    tot = tot + part;
                }
                float mean = tot / (float)N;
                int64_t o = (b * H + h) * D + d;
                if (out_dtype == DT_F16) ((uint16_t*)out)[o] = f32_to_f16(mean);
                else if (out_dtype == DT_BF16) ((uint16_t*)out)[o] = f32_to_bf16(mean);
                else ((float*)out)[o] = mean;
            }
    return 0;
}

/*
 * The attention kernel's arithmetic, one 128-row program at a time (:88-127), KV tiles of 64
 * (:20-72).  mask_kind: 0 none, 1 bool (uint8), 2 additive fp32; mask strides in elements
 * (b, h, m, n), 0 = broadcast.  causal != 0 adds the bottom-right aligned bool mask
 * n <= m + (N - M), treated like an explicit bool mask (tile skip + -1e6).
 * out: fp32 through (os_b, os_h, os_n); lse (may be NULL): [B,Hq,M] base-2.
 * p_dtype: 16-bit type P is rounded to before the PV product (:65); DT_F32 = no rounding.
 * Threads: OpenMP over (b, h, q-block) when compiled with -fopenmp.
 */
int sage_oracle_attn(const int8_t* q, const int8_t* k, const void* v, int v_dtype, const float* q_scale,
                     const float* k_scale, float* out, float* lse, int64_t B, int64_t Hq, int64_t Hkv, int64_t M,
                     int64_t N, int64_t D, int64_t qs_b, int64_t qs_h, int64_t qs_n, int64_t ks_b, int64_t ks_h,
                     int64_t ks_n, int64_t vs_b, int64_t vs_h, int64_t vs_n, int64_t os_b, int64_t os_h,
                     int64_t os_n, const void* mask, int mask_kind, int64_t ms_b, int64_t ms_h, int64_t ms_m,
                     int64_t ms_n, int causal, int p_dtype) {
    const int BM = 128, BN = 64;
    int64_t nq = (M + BM - 1) / BM, nk = (N + BN - 1) / BN, groups = Hq / Hkv;
    int64_t total = B * Hq * nq;
    int err = 0;
#pragma omp parallel for schedule(dynamic)
    for (int64_t job = 0; job < total; job++) {
        int64_t b = job / (Hq * nq), h = (job / nq) % Hq, iq = job % nq, hk = h / groups;
        int64_t m0 = iq * BM, rows = M - m0 < BM ? M - m0 : BM;
        float* acc = (float*)calloc((size_t)(BM * D), sizeof(float));
        float* s = (float*)malloc(sizeof(float) * BM * BN);
        float* vt = (float*)malloc(sizeof(float) * BN * (size_t)D);
        float m_i[128], l_i[128];
        if (!acc || !s || !vt) { err = -1; free(acc); free(s); free(vt); continue; }
        for (int r = 0; r < BM; r++) { m_i[r] = -INFINITY; l_i[r] = 1.0f; } /* :110-111 */
        float sq = q_scale[(b * Hq + h) * nq + iq];
        for (int64_t jk = 0; jk < nk; jk++) {
            int64_t n0 = jk * BN, cols = N - n0 < BN ? N - n0 : BN;
            int use_bool = (mask_kind == 1) || causal;
            if (use_bool) { /* :33-36 skip a tile whose bool mask is False everywhere (OOB loads as False) */
                int any = 0;
                for (int64_t r = 0; r < rows && !any; r++)
                    for (int64_t c = 0; c < cols && !any; c++) {
                        int ok = 1;
                        if (causal) ok = (n0 + c) <= (m0 + r) + (N - M);
                        if (ok && mask_kind == 1)
                            ok = ((const uint8_t*)mask)[b * ms_b + h * ms_h + (m0 + r) * ms_m + (n0 + c) * ms_n] != 0;
                        any |= ok;
                    }
                if (!any) continue;
            }
            float sk = k_scale[(b * Hkv + hk) * nk + jk];
            float sc = sq * sk; /* :44 product of the two scalars first */
            for (int64_t c = 0; c < cols; c++)
                for (int64_t d = 0; d < D; d++)
                    vt[c * D + d] = load_elem(v, v_dtype, b * vs_b + hk * vs_h + (n0 + c) * vs_n + d);
            for (int64_t r = 0; r < rows; r++) {
                const int8_t* qr = q + b * qs_b + h * qs_h + (m0 + r) * qs_n;
                float rmax = -INFINITY;
                for (int64_t c = 0; c < BN; c++) {
                    float x;
                    if (c < cols) {
                        const int8_t* kr = k + b * ks_b + hk * ks_h + (n0 + c) * ks_n;
                        int32_t dot = 0;
                        for (int64_t d = 0; d < D; d++) dot += (int32_t)qr[d] * (int32_t)kr[d];
                        x = (float)dot * sc;
                        if (use_bool) {
                            int ok = 1;
                            if (causal) ok = (n0 + c) <= (m0 + r) + (N - M);
                            if (ok && mask_kind == 1)
                                ok = ((const uint8_t*)mask)[b * ms_b + h * ms_h + (m0 + r) * ms_m + (n0 + c) * ms_n] != 0;
                            x = x + (ok ? 0.0f : -1.0e6f); /* :48 */
                        }
                        if (mask_kind == 2)
                            x = x + ((const float*)mask)[b * ms_b + h * ms_h + (m0 + r) * ms_m + (n0 + c) * ms_n]; /* :50 */
                    } else {
                        x = 0.0f + -1.0e6f; /* masked K loads give 0; :38 / :48 / :52 add -1e6 */
                    }
                    s[r * BN + c] = x;
                    if (x > rmax) rmax = x;
                }
                float m_new = m_i[r] > rmax ? m_i[r] : rmax; /* :54 */
                float l_new = 0.0f;
                for (int64_t c = 0; c < BN; c++) {
                    float p = exp2f(s[r * BN + c] - m_new); /* :55-56 */
                    l_new += p;                            /* :57 fp32 sum of the unrounded P */
                    s[r * BN + c] = round_to(p, p_dtype);  /* :65 */
                }
                float alpha = exp2f(m_i[r] - m_new); /* :59 */
                l_i[r] = l_i[r] * alpha + l_new;     /* :60 */
                float* a = acc + r * D;
                for (int64_t d = 0; d < D; d++) a[d] *= alpha; /* :62 */
                for (int64_t c = 0; c < cols; c++) {
                    float p = s[r * BN + c];
                    const float* vr = vt + c * D;
                    for (int64_t d = 0; d < D; d++) a[d] += p * vr[d]; /* :67 (fp32 accumulate) */
                }
                m_i[r] = m_new;
            }
        }
        for (int64_t r = 0; r < rows; r++) {
            float* o = out + b * os_b + h * os_h + (m0 + r) * os_n;
            for (int64_t d = 0; d < D; d++) o[d] = acc[r * D + d] / l_i[r]; /* :121 */
            if (lse) lse[(b * Hq + h) * M + m0 + r] = log2f(l_i[r]) + m_i[r]; /* :126 */
        }
        free(acc); free(s); free(vt);
    }
    return err;
}

/* conversions exported so the tests can check them against torch's */
uint16_t sage_oracle_f32_to_f16(float f) { return f32_to_f16(f); }
uint16_t sage_oracle_f32_to_bf16(float f) { return f32_to_bf16(f); }
float sage_oracle_f16_to_f32(uint16_t h) { return f16_to_f32(h); }
