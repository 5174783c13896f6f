// Shared host/device helpers of libvlgpu (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/vlgpu.h"

#define VL_EXPORT extern "C" __attribute__((visibility("default")))

constexpr int kWave = 64;

// ---- error plumbing (thread local text, negative return codes) -----------
void vl_set_error(const char *fmt, ...);

#define VL_REQUIRE(cond, ...)                 \
    do {                                      \
        if (!(cond)) {                        \
            vl_set_error(__VA_ARGS__);        \
            return VL_ERR_ARG;                \
        }                                     \
    } while (0)

#define VL_HIP(call)                                                         \
    do {                                                                     \
        hipError_t e_ = (call);                                              \
        if (e_ != hipSuccess) {                                              \
            vl_set_error("%s failed: %s", #call, hipGetErrorString(e_));     \
            return VL_ERR_HIP;                                               \
        }                                                                    \
    } while (0)

#define VL_LAUNCH_CHECK(name)                                                \
    do {                                                                     \
        hipError_t e_ = hipGetLastError();                                   \
        if (e_ != hipSuccess) {                                              \
            vl_set_error("launch of %s failed: %s", name, hipGetErrorString(e_)); \
            return VL_ERR_HIP;                                               \
        }                                                                    \
    } while (0)

// ---- launch size ----------------------------------------------------------
// A grid of 2^32 threads or more in x is not launched whole and no error is
// raised for it, so launchers cut their work into pieces of at most
// kMaxBlocks workgroups (of up to 1024 threads each) and kernels take the
// index of their first row as an argument.
constexpr int64_t kMaxBlocks = 1ll << 21;
// workgroups for an elementwise kernel that strides over n items by its grid size
static inline unsigned vl_grid_for(int64_t n, int per_block) {
    int64_t b = (n + per_block - 1) / per_block;
    return (unsigned)(b < 1 ? 1 : (b > kMaxBlocks ? kMaxBlocks : b));
}

// ---- LDS ---------------------------------------------------------------------
// A gfx950 compute unit has 160 KiB of LDS and a workgroup may take all of it, but a launch that asks for
// more dynamic LDS than the 64 KiB every kernel is allowed by default has to raise that kernel's limit first.
constexpr size_t kLdsDefault = 64 * 1024;
constexpr size_t kLdsPerCu = 160 * 1024;
template <class Kernel>
static inline hipError_t vl_allow_lds(Kernel kernel, size_t smem) {
    if (smem + 1024 <= kLdsDefault) return hipSuccess;  // 1 KiB of slack for the kernels' static LDS
    return hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                               (int)smem);
}

// ---- sort keys -------------------------------------------------------------
// A queue slot is ordered by (distance asc, id asc).  The 64-bit key holds an
// order-preserving image of the float in the high word and the id in the low
// word, so one unsigned compare orders slots.  -0.0 is folded onto +0.0 and
// every NaN onto the positive quiet NaN (sorts after everything, as torch.sort
// places it).
__host__ __device__ inline uint32_t vl_float_key(float d) {
    uint32_t u = __builtin_bit_cast(uint32_t, d);
    if (d != d) u = 0x7FC00000u;
    if (u == 0x80000000u) u = 0u;
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__host__ __device__ inline float vl_key_float(uint32_t k) {
    uint32_t u = (k & 0x80000000u) ? (k & 0x7FFFFFFFu) : ~k;
    return __builtin_bit_cast(float, u);
}
__host__ __device__ inline uint64_t vl_make_key(int32_t id, float d) {
    return ((uint64_t)vl_float_key(d) << 32) | (uint32_t)id;
}
__host__ __device__ inline int32_t vl_key_id(uint64_t k) { return (int32_t)(uint32_t)k; }
__host__ __device__ inline float vl_key_dist(uint64_t k) { return vl_key_float((uint32_t)(k >> 32)); }

constexpr uint64_t kPadKey = ~0ull;  // sorts after every real or empty slot

static inline int vl_next_pow2(int64_t x) {
    int p = 1;
    while (p < x) p <<= 1;
    return p;
}
