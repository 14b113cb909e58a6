#include "common.hpp"

#include <cstring>
#include <mutex>

extern "C" const unsigned char rlx_blob_dequant[], rlx_blob_fakequant[], rlx_blob_gemm[], rlx_blob_gemm_big[], rlx_blob_gemv[], rlx_blob_gemv_wide[], rlx_blob_moe[], rlx_blob_rowops[],
    rlx_blob_topk[];

namespace rlx {

int static_scratch_ptr(void **ptr);  // host/static_scratch.hip

static thread_local std::string g_error;

void set_error(const char *fmt, ...) {
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_error = buf;
}
void clear_error() { g_error.clear(); }
const char *last_error_cstr() { return g_error.c_str(); }

static const char *const kKernelNames[K_COUNT] = {
    "rlx_dequant_q4_0", "rlx_dequant_q8_0", "rlx_dequant_q4_k", "rlx_dequant_q6_k", "rlx_dequant_q5_k", "rlx_dequant_q8_k", "rlx_dequant_q2_k",
    "rlx_fq_col_absmax", "rlx_fq_seg_absmax", "rlx_fq_flat_absmax", "rlx_fq_scale", "rlx_fq_scale_parts", "rlx_fq_col_apply", "rlx_fq_col_apply_img",
    "rlx_fq_flat_apply", "rlx_fq_flat4_apply",
    "rlx_fill_u32", "rlx_copy_u128",
    "rlx_gemv_q4_0_r2", "rlx_gemv_q4_0_r4", "rlx_gemv_q4_0_r2_argmax", "rlx_gemv_q4_0_r2_paired", "rlx_gemv_q4_0_r4_paired",
    "rlx_gemv_q4_0_r2_norm", "rlx_gemv_q4_0_r4_norm", "rlx_gemv_q4_0_r2_norm_paired", "rlx_gemv_q4_0_r4_norm_paired", "rlx_gemv_q4_0_r2_norm_argmax",
    "rlx_gemv_q8_0_r2", "rlx_gemv_q8_0_r4", "rlx_gemv_q8_0_r2_argmax", "rlx_gemv_q8_0_r2_paired", "rlx_gemv_q8_0_r4_paired",
    "rlx_gemv_q8_0_r2_norm", "rlx_gemv_q8_0_r4_norm", "rlx_gemv_q8_0_r2_norm_paired", "rlx_gemv_q8_0_r4_norm_paired", "rlx_gemv_q8_0_r2_norm_argmax",
    "rlx_gemv_q4_k_r2", "rlx_gemv_q4_k_r4", "rlx_gemv_q4_k_r2_argmax", "rlx_gemv_q4_k_r2_paired", "rlx_gemv_q4_k_r4_paired",
    "rlx_gemv_q4_k_r2_norm", "rlx_gemv_q4_k_r4_norm", "rlx_gemv_q4_k_r2_norm_paired", "rlx_gemv_q4_k_r4_norm_paired", "rlx_gemv_q4_k_r2_norm_argmax",
    "rlx_gemv_q6_k_r2", "rlx_gemv_q6_k_r4", "rlx_gemv_q6_k_r2_argmax", "rlx_gemv_q6_k_r2_paired", "rlx_gemv_q6_k_r4_paired",
    "rlx_gemv_q6_k_r2_norm", "rlx_gemv_q6_k_r4_norm", "rlx_gemv_q6_k_r2_norm_paired", "rlx_gemv_q6_k_r4_norm_paired", "rlx_gemv_q6_k_r2_norm_argmax",
    "rlx_gemv_q5_k_r2", "rlx_gemv_q5_k_r4", "rlx_gemv_q5_k_r2_argmax", "rlx_gemv_q5_k_r2_paired", "rlx_gemv_q5_k_r4_paired",
    "rlx_gemv_q5_k_r2_norm", "rlx_gemv_q5_k_r4_norm", "rlx_gemv_q5_k_r2_norm_paired", "rlx_gemv_q5_k_r4_norm_paired", "rlx_gemv_q5_k_r2_norm_argmax",
    "rlx_gemv_q8_k_r2", "rlx_gemv_q8_k_r4", "rlx_gemv_q8_k_r2_argmax", "rlx_gemv_q8_k_r2_paired", "rlx_gemv_q8_k_r4_paired",
    "rlx_gemv_q8_k_r2_norm", "rlx_gemv_q8_k_r4_norm", "rlx_gemv_q8_k_r2_norm_paired", "rlx_gemv_q8_k_r4_norm_paired", "rlx_gemv_q8_k_r2_norm_argmax",
    "rlx_gemv_q2_k_r2", "rlx_gemv_q2_k_r4", "rlx_gemv_q2_k_r2_argmax", "rlx_gemv_q2_k_r2_paired", "rlx_gemv_q2_k_r4_paired",
    "rlx_gemv_q2_k_r2_norm", "rlx_gemv_q2_k_r4_norm", "rlx_gemv_q2_k_r2_norm_paired", "rlx_gemv_q2_k_r4_norm_paired", "rlx_gemv_q2_k_r2_norm_argmax",
    "rlx_gemv_q4_0_u2_r2", "rlx_gemv_q4_0_u2_r4", "rlx_gemv_q4_0_u2_r2_argmax", "rlx_gemv_q4_0_u2_r2_paired", "rlx_gemv_q4_0_u2_r4_paired",
    "rlx_gemv_q4_0_u2_r2_norm", "rlx_gemv_q4_0_u2_r4_norm", "rlx_gemv_q4_0_u2_r2_norm_paired", "rlx_gemv_q4_0_u2_r4_norm_paired", "rlx_gemv_q4_0_u2_r2_norm_argmax",
    "rlx_gemv_q4_0_g2", "rlx_gemv_q8_0_g2", "rlx_gemv_q4_k_g2", "rlx_gemv_q6_k_g2", "rlx_gemv_q5_k_g2", "rlx_gemv_q8_k_g2", "rlx_gemv_q2_k_g2",
    "rlx_gemm_q4_k", "rlx_gemm_q4_0", "rlx_gemm_q8_0", "rlx_gemm64_q4_k", "rlx_gemm64_q4_0", "rlx_gemm64_q8_0", "rlx_gemm_q6_k", "rlx_gemm64_q6_k", "rlx_gemm_q5_k", "rlx_gemm64_q5_k", "rlx_xprep", "rlx_xrowscale", "rlx_argmax_finish", "rlx_topk_select", "rlx_rmsnorm_rows", "rlx_swiglu_rows",
    "rlx_gemm64g_q4_k", "rlx_gemm64g_q4_0", "rlx_gemm64g_q8_0", "rlx_gemm64g_q5_k", "rlx_gemm64g_q6_k", "rlx_moe_sort",
    "rlx_gemm_q8_k", "rlx_gemm64_q8_k", "rlx_gemm64g_q8_k", "rlx_gemm_q2_k", "rlx_gemm64_q2_k", "rlx_gemm64g_q2_k",
    "rlx_gemm_f16w", "rlx_gemm64_f16w", "rlx_wscale_q4_0", "rlx_wscale_q8_0", "rlx_splitk_reduce", "rlx_gemm_big_f16w", "rlx_gemvw_q4_0", "rlx_gemvw_q8_0", "rlx_gemvwg_q4_0", "rlx_gemvwg_q8_0",
};

static std::once_flag g_once;
static int g_init_rc = RLX_ERR_NO_DEVICE;
static std::string g_init_error;
static const unsigned char *const kBlobs[] = {rlx_blob_dequant, rlx_blob_fakequant, rlx_blob_gemm, rlx_blob_gemm_big, rlx_blob_gemv, rlx_blob_gemv_wide,
                                              rlx_blob_moe,     rlx_blob_rowops,    rlx_blob_topk};
constexpr int kModules = (int)(sizeof kBlobs / sizeof kBlobs[0]);
static hipModule_t g_module[kModules];
static hipFunction_t g_fn[K_COUNT];
static DeviceProps g_props;

static int do_init() {
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count <= 0) {
        set_error("no HIP device (hipGetDeviceCount: %s, count=%d)", hipGetErrorString(e), count);
        return RLX_ERR_NO_DEVICE;
    }
    RLX_HIP(hipSetDevice(0));
    hipDeviceProp_t p;
    RLX_HIP(hipGetDeviceProperties(&p, 0));
    if (strncmp(p.gcnArchName, "gfx950", 6) != 0) {
        set_error("device 0 is %s (%s); this library carries gfx950 code only", p.name, p.gcnArchName);
        return RLX_ERR_NO_DEVICE;
    }
    g_props.cu_count = p.multiProcessorCount;
    g_props.clock_khz = p.clockRate;
    g_props.mem_clock_khz = p.memoryClockRate;
    g_props.lds_per_block = p.sharedMemPerBlock;
    snprintf(g_props.arch, sizeof g_props.arch, "%s", p.gcnArchName);
    snprintf(g_props.name, sizeof g_props.name, "%s", p.name);
    for (int m = 0; m < kModules; m++) RLX_HIP(hipModuleLoadData(&g_module[m], kBlobs[m]));
    for (int i = 0; i < K_COUNT; i++) {
        hipError_t fe = hipErrorNotFound;  // a kernel lives in exactly one of the code objects
        for (int m = 0; m < kModules && fe != hipSuccess; m++) fe = hipModuleGetFunction(&g_fn[i], g_module[m], kKernelNames[i]);
        (void)hipGetLastError();
        if (fe != hipSuccess) {
            set_error("hipModuleGetFunction(%s): %s", kKernelNames[i], hipGetErrorString(fe));
            return RLX_ERR_HIP;
        }
    }
    // The array behind rlx_mi355x_fake_quantize_noalloc: looking its address up loads the code object that holds it, which
    // allocates; done here, once, so that the entry point itself only reads the cached pointer.
    void *scratch = nullptr;
    RLX_TRY(static_scratch_ptr(&scratch));
    return RLX_OK;
}

int runtime_init() {
    std::call_once(g_once, [] {
        g_init_rc = do_init();
        if (g_init_rc != RLX_OK) g_init_error = last_error_cstr();
    });
    if (g_init_rc != RLX_OK) set_error("%s", g_init_error.c_str());
    return g_init_rc;
}

const DeviceProps &device_props() { return g_props; }

int launch3(KernelId id, unsigned gx, unsigned gy, unsigned gz, unsigned bx, unsigned shmem, hipStream_t stream,
            void **params) {
    RLX_TRY(runtime_init());
    if (gx == 0 || gy == 0 || gz == 0 || bx == 0 || bx > 1024 || gy > 65535 || gz > 65535 || shmem > 160 * 1024) {
        set_error("launch(%s): bad geometry grid=(%u,%u,%u) block=%u lds=%u", kKernelNames[id], gx, gy, gz, bx, shmem);
        return RLX_ERR_INVALID;
    }
    hipError_t e = hipModuleLaunchKernel(g_fn[id], gx, gy, gz, bx, 1, 1, shmem, stream, params, nullptr);
    if (e != hipSuccess) {
        set_error("hipModuleLaunchKernel(%s, grid=(%u,%u,%u), block=%u, lds=%u): %s", kKernelNames[id], gx, gy, gz, bx,
                  shmem, hipGetErrorString(e));
        return RLX_ERR_HIP;
    }
    return RLX_OK;
}

int launch(KernelId id, unsigned gx, unsigned gy, unsigned bx, unsigned shmem, hipStream_t stream, void **params) {
    return launch3(id, gx, gy, 1, bx, shmem, stream, params);
}

}  // namespace rlx

namespace rlx { const char *last_error_cstr(); }

extern "C" {

int rlx_mi355x_is_available(void) { return rlx::runtime_init() == RLX_OK ? 1 : 0; }
const char *rlx_mi355x_device_name(void) { return "MI355X"; }
int rlx_mi355x_abi_version(void) { return RLX_MI355X_ABI_VERSION; }
const char *rlx_mi355x_last_error(void) { return rlx::last_error_cstr(); }

int rlx_mi355x_device_info(char *buf, size_t cap) {
    RLX_TRY(rlx::runtime_init());
    const rlx::DeviceProps &p = rlx::device_props();
    snprintf(buf, cap, "%s (%s), %d CUs, %.0f MHz core, %.0f MHz mem, %zu B LDS/block", p.name, p.arch, p.cu_count,
             p.clock_khz / 1000.0, p.mem_clock_khz / 1000.0, p.lds_per_block);
    return RLX_OK;
}

int rlx_mi355x_malloc(void **dptr, size_t nbytes) {
    RLX_TRY(rlx::runtime_init());
    RLX_HIP(hipMalloc(dptr, nbytes ? nbytes : 1));
    return RLX_OK;
}
int rlx_mi355x_free(void *dptr) {
    RLX_HIP(hipFree(dptr));
    return RLX_OK;
}
int rlx_mi355x_memcpy_h2d(void *dst, const void *src, size_t nbytes) {
    RLX_HIP(hipMemcpy(dst, src, nbytes, hipMemcpyHostToDevice));
    return RLX_OK;
}
int rlx_mi355x_memcpy_d2h(void *dst, const void *src, size_t nbytes) {
    RLX_HIP(hipMemcpy(dst, src, nbytes, hipMemcpyDeviceToHost));
    return RLX_OK;
}
int rlx_mi355x_memset_u32(void *dst, uint32_t value, size_t n_words, void *stream) {
    if (n_words == 0) return RLX_OK;
    long long n = (long long)n_words;
    unsigned blocks = (unsigned)((n + 255) / 256 > 4096 ? 4096 : (n + 255) / 256);
    void *params[] = {&dst, &value, &n};
    return rlx::launch(rlx::K_FILL_U32, blocks, 1, 256, 0, (hipStream_t)stream, params);
}
int rlx_mi355x_memcpy_d2d(void *dst, const void *src, size_t nbytes, void *stream) {
    if (nbytes == 0) return RLX_OK;
    if ((nbytes | (uintptr_t)dst | (uintptr_t)src) & 15) {
        rlx::set_error("memcpy_d2d: pointers and size must be multiples of 16 bytes");
        return RLX_ERR_INVALID;
    }
    long long n = (long long)(nbytes / 16);
    unsigned blocks = (unsigned)((n + 255) / 256 > 8192 ? 8192 : (n + 255) / 256);
    void *params[] = {&dst, &src, &n};
    return rlx::launch(rlx::K_COPY_U128, blocks, 1, 256, 0, (hipStream_t)stream, params);
}
int rlx_mi355x_stream_create(void **stream) {
    RLX_TRY(rlx::runtime_init());
    hipStream_t s;
    RLX_HIP(hipStreamCreate(&s));  // default priority
    *stream = s;
    return RLX_OK;
}
int rlx_mi355x_stream_destroy(void *stream) {
    RLX_HIP(hipStreamDestroy((hipStream_t)stream));
    return RLX_OK;
}
int rlx_mi355x_stream_sync(void *stream) {
    RLX_HIP(hipStreamSynchronize((hipStream_t)stream));
    return RLX_OK;
}
int rlx_mi355x_event_create(void **event) {
    RLX_TRY(rlx::runtime_init());
    hipEvent_t ev;
    RLX_HIP(hipEventCreate(&ev));
    *event = ev;
    return RLX_OK;
}
int rlx_mi355x_event_destroy(void *event) {
    RLX_HIP(hipEventDestroy((hipEvent_t)event));
    return RLX_OK;
}
int rlx_mi355x_event_record(void *event, void *stream) {
    RLX_HIP(hipEventRecord((hipEvent_t)event, (hipStream_t)stream));
    return RLX_OK;
}
int rlx_mi355x_event_elapsed_ms(void *start, void *stop, float *ms) {
    RLX_HIP(hipEventSynchronize((hipEvent_t)stop));
    RLX_HIP(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
    return RLX_OK;
}

}  // extern "C"
