// Shared host-side helpers of libsage_attention_hip.so (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/sage_attention_hip.h"

namespace sage {

// Records a printf-style message for sage_hip_last_error() and returns `code`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

inline int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(SAGE_E_LAUNCH, "%s: %s", what, hipGetErrorString(e));
    return SAGE_OK;
}

inline int dtype_bytes(int dt) { return dt == SAGE_F32 ? 4 : 2; }

// Launchers implemented in the .hip files.
int launch_quant(const sage_quant_params& p, hipStream_t stream);
int launch_kmean(const sage_tensor& k, int k_dtype, void* km_out, int out_dtype, int64_t B, int64_t H, int64_t N,
                 int64_t D, void* workspace, hipStream_t stream);
int launch_smooth_quant(const sage_quant_params& p, void* km_out, float* q_dot_km, void* workspace, hipStream_t stream);
// Device address of the library's static scratch array on the current device (SAGE_K_MEAN_NOALLOC_MAX_WORKSPACE_BYTES).
int static_scratch(void** out);
// workspace: device memory for the partial results of a key split, or null (then the keys are never split);
// *_split_workspace_bytes: what the launch would use of it (0: it would not split)
int launch_attn(const sage_attn_params& p, void* workspace, int64_t workspace_bytes, hipStream_t stream);
int launch_flash_attn(const sage_flash_params& p, void* workspace, int64_t workspace_bytes, hipStream_t stream);
int64_t attn_split_workspace_bytes(const sage_attn_params& p);
int64_t flash_split_workspace_bytes(const sage_flash_params& p);
int launch_flash_total_attention(const sage_flash_params& p, const float* log_normalizer, float* total, hipStream_t stream);
int launch_flash_dropout(const sage_flash_params& p, float dropout_p, uint64_t seed, uint64_t offset, hipStream_t stream);
int launch_dropout_mask(uint8_t* mask, int64_t count, float dropout_p, uint64_t seed, uint64_t offset, hipStream_t stream);

}  // namespace sage
