// Key split of the pipelined attention kernel for gfx950: planning, and the kernel that combines the partial
// results.  A launch with few (batch, head, q-block) items leaves most of the 256 compute units idle; the keys of
// every item are then cut into `nsplit` runs of whole 64-key steps, one workgroup each, which write a normalized
// fp32 partial output o_s and its base-2 log-sum-exp lse_s.  The combine kernel forms
//     lse = log2 sum_s 2^lse_s,      out = sum_s 2^(lse_s - lse) o_s
// (FlagAttention src/flag_attn/flash.py:73-75, :106-141 is the dense forward's use of the same idea,
// split_kv.py:250-278 its choice of the number of runs, :155-214 its combine kernel).
#include "attn_common.h"

namespace sage {
namespace attn {
namespace {

constexpr int kComputeUnits = 256;
constexpr int kMaxSplits = 64;
constexpr int kMinStepsPerSplit = 4;   // 256 keys: below that the prologue and epilogue of a workgroup dominate
constexpr float kFixedSteps = 6.0f;    // what a workgroup spends outside its step loop, in steps

struct CombineArgs {
    const float* part_o;    // [nsplit, rows, D]
    const float* part_lse;  // [nsplit, rows], base 2
    void* out;
    float* lse;             // [rows] or null
    int64_t os_b, os_h, os_n;
    int64_t rows;           // batch * heads_q * qo_len
    int32_t Hq, M, nsplit, out_dt;
    float lse_mul;
};

constexpr int kCombineThreads = 256;

// One thread per four channels of one row; the threads of a row read the same nsplit log-sum-exps.
template <int D>
__global__ __launch_bounds__(kCombineThreads) void split_combine_kernel(CombineArgs a) {
    constexpr int TPR = D / 4;  // threads per row
    const int64_t row = (int64_t)blockIdx.x * (kCombineThreads / TPR) + threadIdx.x / TPR;
    const int c = threadIdx.x % TPR;
    if (row >= a.rows) return;
    const float* pl = a.part_lse + row;
    float m = -INFINITY;
    for (int s = 0; s < a.nsplit; s++) m = fmaxf(m, pl[(int64_t)s * a.rows]);
    v4f acc = {0.0f, 0.0f, 0.0f, 0.0f};
    float den = 0.0f;
    if (m > -INFINITY) {  // (a row that saw no key in any run: every partial is 0 and every lse_s -inf)
        const float* po = a.part_o + row * D + 4 * c;
#pragma unroll 4
        for (int s = 0; s < a.nsplit; s++) {
            const float w = __builtin_amdgcn_exp2f(pl[(int64_t)s * a.rows] - m);
            const v4f o = *reinterpret_cast<const v4f*>(po + (int64_t)s * a.rows * D);
            den += w;
#pragma unroll
            for (int i = 0; i < 4; i++) acc[i] = __builtin_fmaf(w, o[i], acc[i]);
        }
    }
    const float inv = den > 0.0f ? 1.0f / den : 0.0f;
    float r[4];
#pragma unroll
    for (int i = 0; i < 4; i++) r[i] = acc[i] * inv;
    const int mi = (int)(row % a.M), h = (int)((row / a.M) % a.Hq);
    const int64_t b = row / ((int64_t)a.M * a.Hq);
    const int64_t o = b * a.os_b + (int64_t)h * a.os_h + (int64_t)mi * a.os_n + 4 * c;
    if (a.out_dt == SAGE_BF16) {
        typedef __bf16 b4 __attribute__((ext_vector_type(4)));
        *reinterpret_cast<b4*>(static_cast<__bf16*>(a.out) + o) = b4{(__bf16)r[0], (__bf16)r[1], (__bf16)r[2], (__bf16)r[3]};
    } else if (a.out_dt == SAGE_F16) {
        typedef _Float16 h4 __attribute__((ext_vector_type(4)));
        *reinterpret_cast<h4*>(static_cast<_Float16*>(a.out) + o) = h4{(_Float16)r[0], (_Float16)r[1], (_Float16)r[2], (_Float16)r[3]};
    } else {
        *reinterpret_cast<v4f*>(static_cast<float*>(a.out) + o) = v4f{r[0], r[1], r[2], r[3]};
    }
    if (a.lse && c == 0) a.lse[row] = (__builtin_log2f(den) + m) * a.lse_mul;  // den = 0: log2(0) + (-inf) = -inf
}

}  // namespace

int plan_key_split(int64_t batch, int64_t heads_q, int64_t qo_len, int64_t kv_len, bool causal) {
    const int64_t nq2 = (qo_len + kFastRows - 1) / kFastRows;
    const int64_t per_head = causal ? (nq2 + 1) / 2 : nq2;  // under the causal flag a workgroup takes two q-blocks
    const int64_t base = batch * heads_q * per_head;
    const int64_t nk = (kv_len + BN - 1) / BN;
    if (base * 5 >= kComputeUnits * 4 || nk < 2 * kMinStepsPerSplit) return 1;
    // cost of a plan in steps: rounds of workgroups over the compute units x (steps of a run + fixed part)
    const int smax = (int)(nk / kMinStepsPerSplit < kMaxSplits ? nk / kMinStepsPerSplit : kMaxSplits);
    float best = 0.0f;
    int best_s = 1;
    for (int s = 1; s <= smax; s++) {
        const int64_t steps = (nk + s - 1) / s;
        const int64_t runs = (nk + steps - 1) / steps;  // runs that hold a key
        if (runs != s) continue;
        const int64_t rounds = (base * s + kComputeUnits - 1) / kComputeUnits;
        const float cost = (float)rounds * ((float)steps + kFixedSteps) + (s > 1 ? 0.25f * (float)s : 0.0f);
        if (s == 1 || cost < 0.95f * best) { best = cost; best_s = s; }
    }
    return best_s;
}

int64_t key_split_workspace_bytes(int nsplit, int64_t batch, int64_t heads_q, int64_t qo_len, int64_t head_dim) {
    if (nsplit <= 1) return 0;
    return (int64_t)nsplit * batch * heads_q * qo_len * (head_dim + 1) * (int64_t)sizeof(float);
}

// Points `a` (a complete description of the unsplit launch) at the workspace and sets the split fields.
void apply_key_split(AttnArgs& a, int nsplit, int64_t batch, int head_dim, void* workspace) {
    const int64_t rows = batch * a.Hq * a.M;
    a.nsplit = nsplit;
    a.split_steps = (a.nk + nsplit - 1) / nsplit;
    a.out = workspace;
    a.out_dt = SAGE_F32;
    a.os_n = head_dim; a.os_h = (int64_t)a.M * head_dim; a.os_b = (int64_t)a.Hq * a.M * head_dim;
    a.out_split_stride = rows * head_dim;
    a.lse = static_cast<float*>(workspace) + (int64_t)nsplit * rows * head_dim;
    a.lse_split_stride = rows;
    a.lse_mul = 1.0f;
}

int launch_split_combine(const AttnArgs& split, const AttnArgs& whole, int head_dim, int64_t batch, hipStream_t stream) {
    CombineArgs c{};
    c.part_o = static_cast<const float*>(split.out);
    c.part_lse = split.lse;
    c.out = whole.out; c.lse = whole.lse;
    c.os_b = whole.os_b; c.os_h = whole.os_h; c.os_n = whole.os_n;
    c.rows = batch * whole.Hq * whole.M;
    c.Hq = whole.Hq; c.M = whole.M; c.nsplit = split.nsplit; c.out_dt = whole.out_dt;
    c.lse_mul = whole.lse_mul;
    const int rows_per_wg = kCombineThreads / (head_dim / 4);
    const int64_t wgs = (c.rows + rows_per_wg - 1) / rows_per_wg;
    if (wgs > 0x7fffffffLL) return fail(SAGE_E_UNSUPPORTED, "split combine: too many rows for one launch");
    dim3 grid((unsigned)wgs), block(kCombineThreads);
    if (head_dim == 128) hipLaunchKernelGGL((split_combine_kernel<128>), grid, block, 0, stream, c);
    else hipLaunchKernelGGL((split_combine_kernel<64>), grid, block, 0, stream, c);
    return check_launch("split_combine_kernel");
}

}  // namespace attn
}  // namespace sage
