// extern "C" surface of libsage_attention_hip.so: argument validation and dispatch only.
#include <stdarg.h>
#include <stdio.h>

#include "common.h"

namespace sage {

static thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

static bool float_dtype_ok(int dt) { return dt == SAGE_F16 || dt == SAGE_BF16 || dt == SAGE_F32; }

}  // namespace sage

using namespace sage;

extern "C" const char* sage_hip_last_error(void) { return g_err; }
extern "C" int sage_hip_abi_version(void) { return SAGE_HIP_ABI_VERSION; }

static int check_quant_params(const sage_quant_params* p);

extern "C" int sage_per_block_int8(const sage_quant_params* p, void* stream) {
    if (int rc = check_quant_params(p)) return rc;
    return launch_quant(*p, (hipStream_t)stream);
}

extern "C" int sage_per_block_int8_smooth_k(const sage_smooth_quant_params* sp, void* stream) {
    if (!sp) return fail(SAGE_E_INVALID, "sage_per_block_int8_smooth_k: null params");
    sage_quant_params p = sp->quant;
    p.km.ptr = nullptr;  // the mean is computed here
    if (int rc = check_quant_params(&p)) return rc;
    if (!p.k.ptr || !sp->km_out || !sp->workspace)
        return fail(SAGE_E_INVALID, "sage_per_block_int8_smooth_k: k, km_out and workspace are required");
    if (p.batch <= 0 || p.heads_kv <= 0 || p.kv_len <= 0)
        return fail(SAGE_E_INVALID, "sage_per_block_int8_smooth_k: batch, heads_kv and kv_len must be positive");
    if (sp->q_dot_km) {
        const int64_t d8 = p.head_dim / 8;
        if (!p.q.ptr) return fail(SAGE_E_INVALID, "sage_per_block_int8_smooth_k: q_dot_km needs q");
        if ((d8 & (d8 - 1)) != 0 || d8 > 64)
            return fail(SAGE_E_UNSUPPORTED, "sage_per_block_int8_smooth_k: q_dot_km needs head_dim 8, 16, ..., 512");
        if (p.heads_kv <= 0 || p.heads_q % p.heads_kv != 0)
            return fail(SAGE_E_INVALID, "sage_per_block_int8_smooth_k: heads_q %lld is not a multiple of heads_kv %lld",
                        (long long)p.heads_q, (long long)p.heads_kv);
    }
    return launch_smooth_quant(p, sp->km_out, sp->q_dot_km, sp->workspace, (hipStream_t)stream);
}

static int check_quant_params(const sage_quant_params* p) {
    if (!p) return fail(SAGE_E_INVALID, "sage_per_block_int8: null params");
    if (p->batch < 0 || p->heads_q < 0 || p->heads_kv < 0 || p->qo_len < 0 || p->kv_len < 0)
        return fail(SAGE_E_INVALID, "sage_per_block_int8: negative size");
    if (p->head_dim <= 0 || p->head_dim % 8 != 0)
        return fail(SAGE_E_UNSUPPORTED, "sage_per_block_int8: head_dim %lld must be a positive multiple of 8",
                    (long long)p->head_dim);
    if (!float_dtype_ok(p->in_dtype)) return fail(SAGE_E_INVALID, "sage_per_block_int8: bad in_dtype %d", p->in_dtype);
    if (p->q.ptr && (p->blkq <= 0 || (int64_t)p->blkq * p->head_dim > 32768))
        return fail(SAGE_E_UNSUPPORTED, "sage_per_block_int8: BLKQ*head_dim = %lld exceeds 32768",
                    (long long)p->blkq * p->head_dim);
    if (p->k.ptr && (p->blkk <= 0 || (int64_t)p->blkk * p->head_dim > 32768))
        return fail(SAGE_E_UNSUPPORTED, "sage_per_block_int8: BLKK*head_dim = %lld exceeds 32768",
                    (long long)p->blkk * p->head_dim);
    if (p->q.ptr && (!p->q_int8.ptr || !p->q_scale)) return fail(SAGE_E_INVALID, "sage_per_block_int8: null Q output");
    if (p->k.ptr && (!p->k_int8.ptr || !p->k_scale)) return fail(SAGE_E_INVALID, "sage_per_block_int8: null K output");
    if (p->km.ptr && p->k.ptr) {  // km belongs to K: a call that quantizes Q only ignores it
        if (!float_dtype_ok(p->km_dtype) || !float_dtype_ok(p->diff_dtype))
            return fail(SAGE_E_INVALID, "sage_per_block_int8: bad km_dtype/diff_dtype");
        if (p->in_dtype == SAGE_F32 && p->diff_dtype != SAGE_F32)
            return fail(SAGE_E_INVALID, "sage_per_block_int8: fp32 K needs diff_dtype fp32");
    }
    return SAGE_OK;
}

extern "C" int64_t sage_k_mean_workspace_bytes(int64_t batch, int64_t heads_kv, int64_t kv_len, int64_t head_dim) {
    int64_t nchunk = (kv_len + 63) / 64;
    return batch * heads_kv * nchunk * head_dim * (int64_t)sizeof(float);
}

extern "C" int sage_k_mean(const sage_tensor* k, int32_t k_dtype, void* km_out, int32_t out_dtype, int64_t batch,
                           int64_t heads_kv, int64_t kv_len, int64_t head_dim, void* workspace, void* stream) {
    if (!k || !k->ptr || !km_out || !workspace) return fail(SAGE_E_INVALID, "sage_k_mean: null pointer");
    if (!float_dtype_ok(k_dtype) || !float_dtype_ok(out_dtype)) return fail(SAGE_E_INVALID, "sage_k_mean: bad dtype");
    if (batch <= 0 || heads_kv <= 0 || kv_len <= 0 || head_dim <= 0)
        return fail(SAGE_E_INVALID, "sage_k_mean: sizes must be positive");
    return launch_kmean(*k, k_dtype, km_out, out_dtype, batch, heads_kv, kv_len, head_dim, workspace,
                        (hipStream_t)stream);
}

extern "C" int sage_k_mean_noalloc(const sage_tensor* k, int32_t k_dtype, void* km_out, int32_t out_dtype, int64_t batch,
                                   int64_t heads_kv, int64_t kv_len, int64_t head_dim, void* stream) {
    if (!k || !k->ptr || !km_out) return fail(SAGE_E_INVALID, "sage_k_mean_noalloc: null pointer");
    if (!float_dtype_ok(k_dtype) || !float_dtype_ok(out_dtype))
        return fail(SAGE_E_INVALID, "sage_k_mean_noalloc: bad dtype");
    if (batch <= 0 || heads_kv <= 0 || kv_len <= 0 || head_dim <= 0)
        return fail(SAGE_E_INVALID, "sage_k_mean_noalloc: sizes must be positive");
    // (each factor bounded first, so the product below cannot overflow)
    const int64_t lim = SAGE_K_MEAN_NOALLOC_MAX_WORKSPACE_BYTES;
    if (batch > lim || heads_kv > lim || kv_len > (lim << 6) || head_dim > lim ||
        batch * heads_kv > lim || batch * heads_kv * ((kv_len + 63) / 64) > lim ||
        sage_k_mean_workspace_bytes(batch, heads_kv, kv_len, head_dim) > lim)
        return fail(SAGE_E_UNSUPPORTED,
                    "sage_k_mean_noalloc: batch %lld x heads %lld x ceil(kv_len %lld / 64) x head_dim %lld fp32 partials "
                    "exceed the built-in %lld-byte scratch; use sage_k_mean with a workspace",
                    (long long)batch, (long long)heads_kv, (long long)kv_len, (long long)head_dim, (long long)lim);
    void* ws = nullptr;
    if (int rc = static_scratch(&ws)) return rc;
    return launch_kmean(*k, k_dtype, km_out, out_dtype, batch, heads_kv, kv_len, head_dim, ws, (hipStream_t)stream);
}

static int check_attn_params(const sage_attn_params* p) {
    if (!p) return fail(SAGE_E_INVALID, "sage_attn_fwd: null params");
    if (!p->q.ptr || !p->k.ptr || !p->v.ptr || !p->out.ptr || !p->q_scale || !p->k_scale)
        return fail(SAGE_E_INVALID, "sage_attn_fwd: null tensor pointer");
    if (p->head_dim != 64 && p->head_dim != 128)
        return fail(SAGE_E_UNSUPPORTED, "sage_attn_fwd: head_dim %lld not supported (64 or 128)",
                    (long long)p->head_dim);
    if (p->batch <= 0 || p->heads_q <= 0 || p->heads_kv <= 0 || p->qo_len <= 0 || p->kv_len <= 0)
        return fail(SAGE_E_INVALID, "sage_attn_fwd: sizes must be positive");
    if (p->heads_q % p->heads_kv != 0)
        return fail(SAGE_E_INVALID, "sage_attn_fwd: heads_q %lld is not a multiple of heads_kv %lld",
                    (long long)p->heads_q, (long long)p->heads_kv);
    if (p->v_dtype != SAGE_F16 && p->v_dtype != SAGE_BF16)
        return fail(SAGE_E_UNSUPPORTED, "sage_attn_fwd: V must be fp16 or bf16");
    if (!float_dtype_ok(p->out_dtype)) return fail(SAGE_E_INVALID, "sage_attn_fwd: bad out_dtype %d", p->out_dtype);
    if (p->mask_kind < SAGE_MASK_NONE || p->mask_kind > SAGE_MASK_F32_PADDED)
        return fail(SAGE_E_INVALID, "sage_attn_fwd: bad mask_kind %d", p->mask_kind);
    if (p->mask_kind != SAGE_MASK_NONE && !p->mask) return fail(SAGE_E_INVALID, "sage_attn_fwd: null mask");
    // 16-byte vector loads: row starts of Q/K (int8) and V (16-bit) must be 16-byte aligned
    auto misaligned = [](const sage_tensor& t, int esz) {
        return ((uintptr_t)t.ptr % 16) != 0 || (t.stride_b * esz) % 16 != 0 || (t.stride_h * esz) % 16 != 0 ||
               (t.stride_n * esz) % 16 != 0;
    };
    if (misaligned(p->q, 1) || misaligned(p->k, 1) || misaligned(p->v, 2))
        return fail(SAGE_E_INVALID, "sage_attn_fwd: q/k/v rows must be 16-byte aligned");
    if (misaligned(p->out, dtype_bytes(p->out_dtype)))
        return fail(SAGE_E_INVALID, "sage_attn_fwd: out rows must be 16-byte aligned");
    return SAGE_OK;
}

static int check_workspace(const char* who, const void* workspace, int64_t workspace_bytes) {
    if (workspace_bytes < 0 || (!workspace && workspace_bytes > 0))
        return fail(SAGE_E_INVALID, "%s: bad workspace (null with a size, or a negative size)", who);
    if ((uintptr_t)workspace % 16 != 0) return fail(SAGE_E_INVALID, "%s: workspace must be 16-byte aligned", who);
    return SAGE_OK;
}

extern "C" int sage_attn_fwd(const sage_attn_params* p, void* stream) {
    if (int rc = check_attn_params(p)) return rc;
    return launch_attn(*p, nullptr, 0, (hipStream_t)stream);
}

extern "C" int64_t sage_attn_fwd_workspace_bytes(const sage_attn_params* p) {
    if (check_attn_params(p)) return -1;
    return attn_split_workspace_bytes(*p);
}

extern "C" int sage_attn_fwd_ws(const sage_attn_params* p, void* workspace, int64_t workspace_bytes, void* stream) {
    if (int rc = check_attn_params(p)) return rc;
    if (int rc = check_workspace("sage_attn_fwd_ws", workspace, workspace_bytes)) return rc;
    return launch_attn(*p, workspace, workspace_bytes, (hipStream_t)stream);
}

static int check_flash_params(const sage_flash_params* p, bool forward);

extern "C" int sage_flash_attn_fwd(const sage_flash_params* p, void* stream) {
    if (int rc = check_flash_params(p, true)) return rc;
    return launch_flash_attn(*p, nullptr, 0, (hipStream_t)stream);
}

extern "C" int64_t sage_flash_attn_fwd_workspace_bytes(const sage_flash_params* p) {
    if (check_flash_params(p, true)) return -1;
    return flash_split_workspace_bytes(*p);
}

extern "C" int sage_flash_attn_fwd_ws(const sage_flash_params* p, void* workspace, int64_t workspace_bytes, void* stream) {
    if (int rc = check_flash_params(p, true)) return rc;
    if (int rc = check_workspace("sage_flash_attn_fwd_ws", workspace, workspace_bytes)) return rc;
    return launch_flash_attn(*p, workspace, workspace_bytes, (hipStream_t)stream);
}

// dropout_p in (0, 1); the element index of the random stream is 32-bit arithmetic in the reference
static int check_dropout(const char* who, float dropout_p, int64_t batch, int64_t heads, int64_t qo_len, int64_t kv_len,
                         uint64_t offset) {
    if (!(dropout_p > 0.0f && dropout_p < 1.0f)) return fail(SAGE_E_INVALID, "%s: dropout_p must lie in (0, 1)", who);
    if (batch <= 0 || heads <= 0 || qo_len <= 0 || kv_len <= 0) return fail(SAGE_E_INVALID, "%s: sizes must be positive", who);
    const int64_t lim = 1LL << 31;
    if (batch >= lim || heads >= lim || qo_len >= lim || kv_len >= lim || batch * heads >= lim ||
        batch * heads * qo_len >= lim || batch * heads * qo_len * kv_len >= lim)
        return fail(SAGE_E_UNSUPPORTED, "%s: batch x heads x qo_len x kv_len must stay below 2^31 (the 32-bit element "
                    "index of the random stream wraps beyond)", who);
    if (offset >= (1ULL << 63)) return fail(SAGE_E_INVALID, "%s: offset must be below 2^63", who);
    return SAGE_OK;
}

extern "C" int sage_flash_attn_fwd_dropout(const sage_flash_params* p, float dropout_p, uint64_t seed, uint64_t offset,
                                           void* stream) {
    if (int rc = check_flash_params(p, true)) return rc;
    if (int rc = check_dropout("sage_flash_attn_fwd_dropout", dropout_p, p->batch, p->heads_q, p->qo_len, p->kv_len, offset))
        return rc;
    return launch_flash_dropout(*p, dropout_p, seed, offset, (hipStream_t)stream);
}

extern "C" int sage_flash_dropout_mask(uint8_t* mask, int64_t batch, int64_t heads_q, int64_t qo_len, int64_t kv_len,
                                       float dropout_p, uint64_t seed, uint64_t offset, void* stream) {
    if (!mask) return fail(SAGE_E_INVALID, "sage_flash_dropout_mask: null mask");
    if (int rc = check_dropout("sage_flash_dropout_mask", dropout_p, batch, heads_q, qo_len, kv_len, offset)) return rc;
    return launch_dropout_mask(mask, batch * heads_q * qo_len * kv_len, dropout_p, seed, offset, (hipStream_t)stream);
}

extern "C" int sage_flash_total_attention(const sage_flash_params* p, const float* log_normalizer, float* total_attention,
                                          void* stream) {
    if (int rc = check_flash_params(p, false)) return rc;
    if (!log_normalizer || !total_attention)
        return fail(SAGE_E_INVALID, "sage_flash_total_attention: null log_normalizer or total_attention");
    return launch_flash_total_attention(*p, log_normalizer, total_attention, (hipStream_t)stream);
}

static int check_flash_params(const sage_flash_params* p, bool forward) {
    if (!p) return fail(SAGE_E_INVALID, "sage_flash_attn_fwd: null params");
    if (!p->q.ptr || !p->k.ptr || (forward && (!p->v.ptr || !p->out.ptr)))
        return fail(SAGE_E_INVALID, "sage_flash_attn_fwd: null tensor pointer");
    if (p->head_dim != 64 && p->head_dim != 128)
        return fail(SAGE_E_UNSUPPORTED, "sage_flash_attn_fwd: head_dim %lld not supported (64 or 128)",
                    (long long)p->head_dim);
    if (p->batch <= 0 || p->heads_q <= 0 || p->heads_kv <= 0 || p->qo_len <= 0 || p->kv_len <= 0)
        return fail(SAGE_E_INVALID, "sage_flash_attn_fwd: sizes must be positive");
    if (p->heads_q % p->heads_kv != 0)
        return fail(SAGE_E_INVALID, "sage_flash_attn_fwd: heads_q %lld is not a multiple of heads_kv %lld",
                    (long long)p->heads_q, (long long)p->heads_kv);
    if (p->dtype != SAGE_F16 && p->dtype != SAGE_BF16)
        return fail(SAGE_E_UNSUPPORTED, "sage_flash_attn_fwd: q, k, v must be fp16 or bf16");
    if (forward && !float_dtype_ok(p->out_dtype)) return fail(SAGE_E_INVALID, "sage_flash_attn_fwd: bad out_dtype %d", p->out_dtype);
    if (!(p->sm_scale > 0.0f) || !(p->sm_scale < 3.0e38f))
        return fail(SAGE_E_INVALID, "sage_flash_attn_fwd: sm_scale must be positive and finite");
    auto misaligned = [](const sage_tensor& t, int esz) {
        return ((uintptr_t)t.ptr % 16) != 0 || (t.stride_b * esz) % 16 != 0 || (t.stride_h * esz) % 16 != 0 ||
               (t.stride_n * esz) % 16 != 0;
    };
    if (misaligned(p->q, 2) || misaligned(p->k, 2) || (forward && misaligned(p->v, 2)))
        return fail(SAGE_E_INVALID, "sage_flash_attn_fwd: q/k/v rows must be 16-byte aligned");
    if (forward && misaligned(p->out, dtype_bytes(p->out_dtype)))
        return fail(SAGE_E_INVALID, "sage_flash_attn_fwd: out rows must be 16-byte aligned");
    return SAGE_OK;
}
