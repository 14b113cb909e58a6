// Host-side plumbing shared by every translation unit of librlx_mi355x.so: error text, HIP call checking,
// the embedded gfx950 code object and the kernel launcher (hipModuleLoadData / hipModuleLaunchKernel only;
// no hipBLAS, MIOpen or runtime compilation anywhere).
#pragma once
#include <hip/hip_runtime_api.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <string>

#include "../../../include/rlx_mi355x.h"
#include "../layout.h"

namespace rlx {

void set_error(const char *fmt, ...) __attribute__((format(printf, 1, 2)));
void clear_error();

// Evaluates a HIP call; on failure records "<call>: <hipGetErrorString>" and returns RLX_ERR_HIP from the caller.
#define RLX_HIP(call)                                                                               \
    do {                                                                                            \
        hipError_t e_ = (call);                                                                     \
        if (e_ != hipSuccess) {                                                                     \
            ::rlx::set_error("%s failed: %s (%d) at %s:%d", #call, hipGetErrorString(e_), (int)e_, \
                             __FILE__, __LINE__);                                                   \
            return RLX_ERR_HIP;                                                                     \
        }                                                                                           \
    } while (0)

#define RLX_TRY(expr)             \
    do {                          \
        int rc_ = (expr);         \
        if (rc_ < 0) return rc_;  \
    } while (0)

enum KernelId : int {
    K_DEQUANT_Q4_0, K_DEQUANT_Q8_0, K_DEQUANT_Q4_K, K_DEQUANT_Q6_K, K_DEQUANT_Q5_K, K_DEQUANT_Q8_K, K_DEQUANT_Q2_K,
    K_FQ_COL_ABSMAX, K_FQ_SEG_ABSMAX, K_FQ_FLAT_ABSMAX, K_FQ_SCALE, K_FQ_SCALE_PARTS, K_FQ_COL_APPLY, K_FQ_COL_APPLY_IMG, K_FQ_FLAT_APPLY, K_FQ_FLAT4_APPLY,
    K_FILL_U32, K_COPY_U128,
    // decode GEMV: per scheme {r2, r4, r2_argmax, r2_paired, r4_paired, r2_norm, r4_norm, r2_norm_paired, r4_norm_paired,
    // r2_norm_argmax}, in this order (launch_gemv indexes into it)
    K_GEMV_Q4_0_R2, K_GEMV_Q4_0_R4, K_GEMV_Q4_0_R2_ARGMAX, K_GEMV_Q4_0_R2_PAIRED, K_GEMV_Q4_0_R4_PAIRED,
    K_GEMV_Q4_0_R2_NORM, K_GEMV_Q4_0_R4_NORM, K_GEMV_Q4_0_R2_NORM_PAIRED, K_GEMV_Q4_0_R4_NORM_PAIRED, K_GEMV_Q4_0_R2_NORM_ARGMAX,
    K_GEMV_Q8_0_R2, K_GEMV_Q8_0_R4, K_GEMV_Q8_0_R2_ARGMAX, K_GEMV_Q8_0_R2_PAIRED, K_GEMV_Q8_0_R4_PAIRED,
    K_GEMV_Q8_0_R2_NORM, K_GEMV_Q8_0_R4_NORM, K_GEMV_Q8_0_R2_NORM_PAIRED, K_GEMV_Q8_0_R4_NORM_PAIRED, K_GEMV_Q8_0_R2_NORM_ARGMAX,
    K_GEMV_Q4_K_R2, K_GEMV_Q4_K_R4, K_GEMV_Q4_K_R2_ARGMAX, K_GEMV_Q4_K_R2_PAIRED, K_GEMV_Q4_K_R4_PAIRED,
    K_GEMV_Q4_K_R2_NORM, K_GEMV_Q4_K_R4_NORM, K_GEMV_Q4_K_R2_NORM_PAIRED, K_GEMV_Q4_K_R4_NORM_PAIRED, K_GEMV_Q4_K_R2_NORM_ARGMAX,
    K_GEMV_Q6_K_R2, K_GEMV_Q6_K_R4, K_GEMV_Q6_K_R2_ARGMAX, K_GEMV_Q6_K_R2_PAIRED, K_GEMV_Q6_K_R4_PAIRED,
    K_GEMV_Q6_K_R2_NORM, K_GEMV_Q6_K_R4_NORM, K_GEMV_Q6_K_R2_NORM_PAIRED, K_GEMV_Q6_K_R4_NORM_PAIRED, K_GEMV_Q6_K_R2_NORM_ARGMAX,
    K_GEMV_Q5_K_R2, K_GEMV_Q5_K_R4, K_GEMV_Q5_K_R2_ARGMAX, K_GEMV_Q5_K_R2_PAIRED, K_GEMV_Q5_K_R4_PAIRED,
    K_GEMV_Q5_K_R2_NORM, K_GEMV_Q5_K_R4_NORM, K_GEMV_Q5_K_R2_NORM_PAIRED, K_GEMV_Q5_K_R4_NORM_PAIRED, K_GEMV_Q5_K_R2_NORM_ARGMAX,
    K_GEMV_Q8_K_R2, K_GEMV_Q8_K_R4, K_GEMV_Q8_K_R2_ARGMAX, K_GEMV_Q8_K_R2_PAIRED, K_GEMV_Q8_K_R4_PAIRED,
    K_GEMV_Q8_K_R2_NORM, K_GEMV_Q8_K_R4_NORM, K_GEMV_Q8_K_R2_NORM_PAIRED, K_GEMV_Q8_K_R4_NORM_PAIRED, K_GEMV_Q8_K_R2_NORM_ARGMAX,
    K_GEMV_Q2_K_R2, K_GEMV_Q2_K_R4, K_GEMV_Q2_K_R2_ARGMAX, K_GEMV_Q2_K_R2_PAIRED, K_GEMV_Q2_K_R4_PAIRED,
    K_GEMV_Q2_K_R2_NORM, K_GEMV_Q2_K_R4_NORM, K_GEMV_Q2_K_R2_NORM_PAIRED, K_GEMV_Q2_K_R4_NORM_PAIRED, K_GEMV_Q2_K_R2_NORM_ARGMAX,
    K_GEMV_Q4_0_U2_R2, K_GEMV_Q4_0_U2_R4, K_GEMV_Q4_0_U2_R2_ARGMAX, K_GEMV_Q4_0_U2_R2_PAIRED, K_GEMV_Q4_0_U2_R4_PAIRED,
    K_GEMV_Q4_0_U2_R2_NORM, K_GEMV_Q4_0_U2_R4_NORM, K_GEMV_Q4_0_U2_R2_NORM_PAIRED, K_GEMV_Q4_0_U2_R4_NORM_PAIRED, K_GEMV_Q4_0_U2_R2_NORM_ARGMAX,
    K_GEMV_Q4_0_G2, K_GEMV_Q8_0_G2, K_GEMV_Q4_K_G2, K_GEMV_Q6_K_G2, K_GEMV_Q5_K_G2, K_GEMV_Q8_K_G2, K_GEMV_Q2_K_G2,
    K_GEMM_Q4_K, K_GEMM_Q4_0, K_GEMM_Q8_0, K_GEMM64_Q4_K, K_GEMM64_Q4_0, K_GEMM64_Q8_0, K_GEMM_Q6_K, K_GEMM64_Q6_K, K_GEMM_Q5_K, K_GEMM64_Q5_K, K_XPREP, K_XROWSCALE, K_ARGMAX_FINISH, K_TOPK_SELECT, K_RMSNORM_ROWS, K_SWIGLU_ROWS,
    K_GEMM64G_Q4_K, K_GEMM64G_Q4_0, K_GEMM64G_Q8_0, K_GEMM64G_Q5_K, K_GEMM64G_Q6_K, K_MOE_SORT,
    K_GEMM_Q8_K, K_GEMM64_Q8_K, K_GEMM64G_Q8_K, K_GEMM_Q2_K, K_GEMM64_Q2_K, K_GEMM64G_Q2_K,
    K_GEMM_F16W, K_GEMM64_F16W, K_WSCALE_Q4_0, K_WSCALE_Q8_0, K_SPLITK_REDUCE, K_GEMM_BIG_F16W, K_GEMVW_Q4_0, K_GEMVW_Q8_0, K_GEMVWG_Q4_0, K_GEMVWG_Q8_0,
    K_COUNT
};

// Loads the embedded code object on first use (device 0). RLX_OK or an error code with text.
int runtime_init();
// Launches kernel `id`; `args` points at the kernel's single by-value argument struct (or packed scalars).
int launch(KernelId id, unsigned gx, unsigned gy, unsigned bx, unsigned shmem, hipStream_t stream, void **params);
int launch3(KernelId id, unsigned gx, unsigned gy, unsigned gz, unsigned bx, unsigned shmem, hipStream_t stream, void **params);

struct DeviceProps {
    int cu_count;
    int clock_khz;
    int mem_clock_khz;
    size_t lds_per_block;
    char arch[64];
    char name[128];
};
const DeviceProps &device_props();

}  // namespace rlx
