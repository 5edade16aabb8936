// Types shared by the attention kernels of libsage_attention_hip.so (gfx950).
#pragma once
#include "common.h"

namespace sage {
namespace attn {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

constexpr int kThreads = 256;
constexpr int BM = 128;  // query rows per workgroup (= Q quantization block)
constexpr int BN = 64;   // keys per step (= K quantization block)
constexpr int kFastRows = 256;  // query rows per workgroup of the pipelined kernel (attn_fast_kernel.h)
constexpr float kMasked = -1.0e6f;
constexpr float kTau = 8.0f;  // log2 of the largest P tolerated before the running maximum is advanced

enum { MODE_PLAIN = 0, MODE_CAUSAL = 1, MODE_MASK_BOOL = 2, MODE_MASK_F32 = 3 };

struct AttnArgs {
    const int8_t* q;
    const int8_t* k;
    const void* v;
    void* out;
    const float* q_scale;
    const float* k_scale;
    float* lse;
    const void* mask;
    int64_t qs_b, qs_h, qs_n;
    int64_t ks_b, ks_h, ks_n;
    int64_t vs_b, vs_h, vs_n;
    int64_t os_b, os_h, os_n;
    int64_t ms_b, ms_h, ms_m, ms_n;
    int32_t Hq, Hkv, M, N, nq, nk, groups;
    int32_t out_dt, causal;
    int32_t total_wg;
    int32_t mask_vec;  // mask rows are contiguous along the keys and every group of four entries is naturally aligned
    int32_t mask_dt;   // storage type of an additive mask (SAGE_F32 / SAGE_F16 / SAGE_BF16)
    int32_t mask_additive;  // the mask tensor is additive (entries of type mask_dt), not bool
    int32_t mask_padded;  // mask rows are readable (bool: and zero) up to the next multiple of 16 bytes past kv_len
    int32_t mask_causal;  // the bool mask is False wherever n > m + (kv_len - qo_len): tiles beyond need no visit
    // Heads that take turns within one q-block in the order of the workgroups (1: a head's q-blocks follow each
    // other).  Under a mask shared by the heads, head_tile heads x several q-blocks run side by side on an XCD, so
    // that both the mask tiles (shared by the heads) and the K/V tiles (shared by the q-blocks) are re-read from L2.
    int32_t head_tile;
    // Split of the keys over several workgroups per (batch, head, q-block) (never under a mask tensor): workgroup s
    // of `nsplit` takes steps s * split_steps .. and writes an fp32 partial output and its base-2 log-sum-exp to
    // out + s * out_split_stride / lse + s * lse_split_stride, which a second kernel combines.  Unsplit: 1, nk, 0, 0.
    int32_t nsplit, split_steps;
    int64_t out_split_stride, lse_split_stride;
    float lse_mul;     // factor on the base-2 log-sum-exp on its way out (1: as is; ln 2: natural log)
    float qk_scale;    // 16-bit Q and K only: sm_scale * log2(e), the one scale of every score (q/k point at 16-bit data)
};

template <typename VT> struct PV;
template <> struct PV<__bf16> {
    typedef bf16x8 vec;
    static __device__ __forceinline__ v16f mfma(vec a, vec b, v16f c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ v4f mfma16(vec a, vec b, v4f c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
    }
    // acc + p[2c] + p[2c+1]
    static __device__ __forceinline__ float dot2_ones(vec p, int c, float acc) {
        typedef __bf16 v2 __attribute__((ext_vector_type(2)));
        const v2 ones = {(__bf16)1.0f, (__bf16)1.0f};
        const v2 pr = {p[2 * c], p[2 * c + 1]};
        return __builtin_amdgcn_fdot2_f32_bf16(pr, ones, acc, false);
    }
};
template <> struct PV<_Float16> {
    typedef f16x8 vec;
    static __device__ __forceinline__ v16f mfma(vec a, vec b, v16f c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ v4f mfma16(vec a, vec b, v4f c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ float dot2_ones(vec p, int c, float acc) {
        typedef _Float16 v2 __attribute__((ext_vector_type(2)));
        const v2 ones = {(_Float16)1.0f, (_Float16)1.0f};
        const v2 pr = {p[2 * c], p[2 * c + 1]};
        return __builtin_amdgcn_fdot2(pr, ones, acc, false);
    }
};


// Launches the software-pipelined kernel: no mask tensor, and qo_len <= kv_len when causal.
// head_dim 64 / 128, V dtype fp16 / bf16.
int launch_fast(const AttnArgs& a, int head_dim, int v_dtype, bool causal, hipStream_t stream);

// Key split for launches that would leave most compute units idle (split_combine.hip).  plan_key_split: how many
// workgroups share the keys of one (batch, head, q-block), 1 when the launch fills the chip anyway.
// apply_key_split turns the arguments of the unsplit launch into those of the split one (partial results in
// `workspace`, key_split_workspace_bytes large); launch_split_combine writes what the unsplit launch would have.
int plan_key_split(int64_t batch, int64_t heads_q, int64_t qo_len, int64_t kv_len, bool causal);
int64_t key_split_workspace_bytes(int nsplit, int64_t batch, int64_t heads_q, int64_t qo_len, int64_t head_dim);
void apply_key_split(AttnArgs& a, int nsplit, int64_t batch, int head_dim, void* workspace);
int launch_split_combine(const AttnArgs& split, const AttnArgs& whole, int head_dim, int64_t batch, hipStream_t stream);

// The same kernel under a bool mask tensor or an additive fp16 / bf16 one, where fast_serves_mask() says so (a.mask
// set; esz: bytes per mask entry).
bool fast_serves_mask(const AttnArgs& a, int esz);
int launch_fast_masked(const AttnArgs& a, int head_dim, int v_dtype, hipStream_t stream);
int launch_fast_additive(const AttnArgs& a, int head_dim, int v_dtype, hipStream_t stream);

// The same kernel on 16-bit Q and K (dense attention); causal with any qo_len / kv_len.
int launch_flash(const AttnArgs& a, int head_dim, int dtype, bool causal, hipStream_t stream);

}  // namespace attn
}  // namespace sage
