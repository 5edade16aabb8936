// Dense attention forward on 16-bit Q, K, V for gfx950: the software-pipelined kernel of
// attn_fast_kernel.h instantiated for 16-bit Q and K (FlagAttention src/flag_attn/flash.py:346-510
// is the kernel it stands in for, :37-180 the host side).  What differs from the int8 instances: the
// Q.K^T product is 2 * head_dim / 16 v_mfma_f32_32x32x16 instructions per 64-key step into fp32
// accumulators, every score has the same scale sm_scale * log2(e), the K tiles are twice as large
// (128 KB of LDS hold four K and four V tiles at head_dim 128), and the causal flag is served for any
// qo_len / kv_len (a query that sees no key ends with l = 0: zero row, log normalizer -inf).
#include "attn_fast_kernel.h"

namespace sage {
namespace attn {
namespace {

template <int D, typename VT>
int launch_dense(const AttnArgs& a, bool hides_keys, hipStream_t stream) {
    const int nq2 = (a.M + kFastRows - 1) / kFastRows;
    AttnArgs b = a;
    const int per_head = a.causal ? (nq2 + 1) / 2 : nq2;  // under the causal flag a workgroup takes two q-blocks
    b.total_wg = (int)((int64_t)a.total_wg / nq2 * per_head) * a.nsplit;
    dim3 grid((unsigned)b.total_wg), block(kFastThreads);
    if (hides_keys) hipLaunchKernelGGL((sage_attn_fwd_fast_kernel<D, VT, true, 2>), grid, block, 0, stream, b, nq2);
    else hipLaunchKernelGGL((sage_attn_fwd_fast_kernel<D, VT, false, 2>), grid, block, 0, stream, b, nq2);
    return check_launch("sage_attn_fwd_fast_kernel (16-bit Q, K)");
}

}  // namespace

int launch_flash(const AttnArgs& a, int head_dim, int dtype, bool causal, hipStream_t stream) {
    const bool hides_keys = causal || (a.N % BN) != 0;  // a ragged last tile has hidden keys too
    if (head_dim == 128)
        return dtype == SAGE_BF16 ? launch_dense<128, __bf16>(a, hides_keys, stream)
                                  : launch_dense<128, _Float16>(a, hides_keys, stream);
    return dtype == SAGE_BF16 ? launch_dense<64, __bf16>(a, hides_keys, stream)
                              : launch_dense<64, _Float16>(a, hides_keys, stream);
}

}  // namespace attn

static int flash_key_splits(const sage_flash_params& p) {
    return attn::plan_key_split(p.batch, p.heads_q, p.qo_len, p.kv_len, p.causal != 0);
}

int64_t flash_split_workspace_bytes(const sage_flash_params& p) {
    return attn::key_split_workspace_bytes(flash_key_splits(p), p.batch, p.heads_q, p.qo_len, p.head_dim);
}

int launch_flash_attn(const sage_flash_params& p, void* workspace, int64_t workspace_bytes, hipStream_t stream) {
    using namespace attn;
    AttnArgs a{};
    a.q = (const int8_t*)p.q.ptr; a.k = (const int8_t*)p.k.ptr; a.v = p.v.ptr; a.out = p.out.ptr;
    a.lse = p.log_normalizer;
    a.qs_b = p.q.stride_b; a.qs_h = p.q.stride_h; a.qs_n = p.q.stride_n;
    a.ks_b = p.k.stride_b; a.ks_h = p.k.stride_h; a.ks_n = p.k.stride_n;
    a.vs_b = p.v.stride_b; a.vs_h = p.v.stride_h; a.vs_n = p.v.stride_n;
    a.os_b = p.out.stride_b; a.os_h = p.out.stride_h; a.os_n = p.out.stride_n;
    a.Hq = (int)p.heads_q; a.Hkv = (int)p.heads_kv; a.M = (int)p.qo_len; a.N = (int)p.kv_len;
    a.nq = (int)((p.qo_len + BM - 1) / BM); a.nk = (int)((p.kv_len + BN - 1) / BN);
    a.groups = (int)(p.heads_q / p.heads_kv);
    a.out_dt = p.out_dtype; a.causal = p.causal ? 1 : 0;
    a.lse_mul = 0.693147180559945309f;         // base-2 log-sum-exp -> natural log
    a.qk_scale = p.sm_scale * 1.44269504089f;  // scores in base-2 units, as the reference kernel does (flash.py:372-373)
    const int64_t total = p.batch * p.heads_q * ((p.qo_len + kFastRows - 1) / kFastRows);
    if (total > 0x7fffffffLL || p.qo_len > 0x7fffffffLL - kFastRows || p.kv_len > 0x7fffffffLL - BN)
        return fail(SAGE_E_UNSUPPORTED, "sage_flash_attn_fwd: problem too large for 32-bit tile indices");
    if (p.k.stride_n < 0 || p.v.stride_n < 0 || (int64_t)BN * p.k.stride_n >= (1LL << 29) ||
        (int64_t)BN * p.v.stride_n >= (1LL << 29))
        return fail(SAGE_E_UNSUPPORTED, "sage_flash_attn_fwd: k/v sequence stride out of range for 32-bit tile offsets");
    a.total_wg = (int)total;
    a.nsplit = 1; a.split_steps = a.nk;
    const int nsplit = workspace ? flash_key_splits(p) : 1;
    if (nsplit > 1 && workspace_bytes >= key_split_workspace_bytes(nsplit, p.batch, p.heads_q, p.qo_len, p.head_dim)) {
        if (total * nsplit > 0x7fffffffLL) return fail(SAGE_E_UNSUPPORTED, "sage_flash_attn_fwd: problem too large for 32-bit tile indices");
        AttnArgs s = a;
        apply_key_split(s, nsplit, p.batch, (int)p.head_dim, workspace);
        if (int rc = launch_flash(s, (int)p.head_dim, p.dtype, p.causal != 0, stream)) return rc;
        return launch_split_combine(s, a, (int)p.head_dim, p.batch, stream);
    }
    return launch_flash(a, (int)p.head_dim, p.dtype, p.causal != 0, stream);
}

}  // namespace sage
