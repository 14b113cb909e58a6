// The one entry point of the library that allocates nothing: FakeQuantize with its scratch (per-channel maxima, scales
// and the partial maxima of the column pass) in a device array that is part of the library image, for callers that
// cannot call hipMalloc (stream capture in progress, tight serving loops, harnesses that forbid allocation).
//
// This file is compiled by hipcc for host and device together (the rest of the host side is plain C++ and the kernels
// are a separate code object): the array below needs a device definition and a host-side handle in one translation unit.
#include <hip/hip_runtime.h>

#include <mutex>

#include "common.hpp"

// 8 MiB per GPU, held until the process ends. The column plan needs 8 bytes per channel plus at most 1024 row blocks x
// 4 bytes per channel of partial maxima: [8192, 4096] takes 4.03 MiB.
#define RLX_FQ_STATIC_SCRATCH_BYTES (8u << 20)

// In host code this name is only a handle for hipGetSymbolAddress, never an address to hand to a kernel.
static __device__ __align__(256) unsigned char scratch[RLX_FQ_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
void *g_scratch_ptr[kMaxDevices];  // per device: that device's copy of the array
std::mutex g_scratch_mutex;
}  // namespace

namespace rlx {

// Device address of the current device's copy of the array, looked up once per device with that device current.
int static_scratch_ptr(void **ptr) {
    int dev = -1;
    RLX_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) {
        set_error("static scratch: device ordinal %d out of range", dev);
        return RLX_ERR_INVALID;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        RLX_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p || ((uintptr_t)p & 255) != 0) {
            set_error("static scratch: hipGetSymbolAddress gave %p", p);
            return RLX_ERR_HIP;
        }
        g_scratch_ptr[dev] = p;
    }
    *ptr = g_scratch_ptr[dev];
    return RLX_OK;
}

}  // namespace rlx

extern "C" {

size_t rlx_mi355x_fake_quantize_noalloc_max_scratch(void) { return RLX_FQ_STATIC_SCRATCH_BYTES; }

int rlx_mi355x_fake_quantize_noalloc(const float *x_dev, float *out_dev, int8_t *codes_dev, int64_t len, int64_t chan_dim,
                                     int64_t inner, int bits, int scale_mode, float ema_decay, float *state_dev, int round_mode,
                                     void *stream) {
    const size_t need = rlx_mi355x_fake_quantize_scratch_bytes(len, chan_dim, inner);
    if (need > RLX_FQ_STATIC_SCRATCH_BYTES) {
        rlx::set_error("fake_quantize_noalloc: this shape needs %zu bytes of scratch, the built-in scratch holds %u; use "
                       "rlx_mi355x_fake_quantize with a scratch buffer of your own",
                       need, RLX_FQ_STATIC_SCRATCH_BYTES);
        return RLX_ERR_UNSUPPORTED;
    }
    RLX_TRY(rlx::runtime_init());
    void *ptr = nullptr;
    RLX_TRY(rlx::static_scratch_ptr(&ptr));
    // Every buffer of the scratch that a pass reads is written by an earlier pass of the same call (the flat and segment
    // passes clear their maxima with a fill kernel first), so nothing a previous call left behind is ever read.
    return rlx_mi355x_fake_quantize(x_dev, out_dev, codes_dev, len, chan_dim, inner, bits, scale_mode, ema_decay, state_dev,
                                    round_mode, ptr, stream);
}

}  // extern "C"
