// Shared device helpers for the gfx950 kernels: storage types, conversions,
// wave and block reductions, and the error slot of the C interface.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#define HB_WAVE 64

// dtype codes of the C interface
#define HB_F32 0
#define HB_BF16 1

// bfloat16 as stored: the upper half of a float32.
struct bf16 {
    uint16_t bits;
};

__device__ __forceinline__ float hb_to_float(float v) { return v; }
__device__ __forceinline__ float hb_to_float(bf16 v) {
    return __uint_as_float(((uint32_t)v.bits) << 16);
}

template <class T> __device__ __forceinline__ T hb_from_float(float v);
template <> __device__ __forceinline__ float hb_from_float<float>(float v) { return v; }
// Round to nearest, ties to even, on the upper 16 bits; NaN stays NaN.
template <> __device__ __forceinline__ bf16 hb_from_float<bf16>(float v) {
    uint32_t u = __float_as_uint(v);
    bf16 r;
    if ((u & 0x7fffffffu) > 0x7f800000u) {
        r.bits = (uint16_t)((u >> 16) | 0x0040u);
        return r;
    }
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    r.bits = (uint16_t)(u >> 16);
    return r;
}

__device__ __forceinline__ float hb_wave_sum(float v) {
#pragma unroll
    for (int off = HB_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, HB_WAVE);
    return v;
}

__device__ __forceinline__ float hb_wave_max(float v) {
#pragma unroll
    for (int off = HB_WAVE / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, HB_WAVE));
    return v;
}

// ---- loads from global memory straight into LDS, and what orders them ----
// global_load_lds_dwordx4: a lane's 16 bytes land at lds_base + 16 * lane (lds_base is uniform);
// no registers, no ds_write. The loads count in vmcnt like any other.
__device__ __forceinline__ void hb_load_to_lds(const void* global_src, void* lds_base) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)global_src,
                                     (__attribute__((address_space(3))) void*)lds_base, 16, 0, 0);
}

template <int N_OUTSTANDING>
__device__ __forceinline__ void hb_wait_vmcnt() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N_OUTSTANDING) : "memory");
}

// The barrier alone: __syncthreads() would first wait for every load in flight, those of later
// stages too. What has to have landed is waited for by hb_wait_vmcnt before it; the reads of
// LDS issued so far are waited for here, so that what they read may be overwritten afterwards.
__device__ __forceinline__ void hb_workgroup_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// Sum over a block of up to 1024 threads; `red` holds one float per wave.
// Every thread gets the result; the order of additions is fixed.
__device__ __forceinline__ float hb_block_sum(float v, float* red) {
    const int lane = threadIdx.x & (HB_WAVE - 1);
    const int wave = threadIdx.x / HB_WAVE;
    const int nwaves = (blockDim.x + HB_WAVE - 1) / HB_WAVE;
    v = hb_wave_sum(v);
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float total = 0.f;
    for (int i = 0; i < nwaves; ++i) total += red[i];
    return total;
}

// ---- error slot of the C interface -------------------------------------
// Every entry point returns 0 on success; otherwise hb_last_error() gives the text.
// Each module (one .hip file built into one shared library) holds a slot of its own.
#include <stdarg.h>
inline char* hb_error_buffer() {
    static thread_local char buf[1024] = {0};
    return buf;
}
inline void hb_set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(hb_error_buffer(), 1024, fmt, ap);
    va_end(ap);
}
#define HB_MODULE_ERROR_SLOT() \
    extern "C" const char* hb_last_error() { return hb_error_buffer(); }

#define HB_REQUIRE(cond, ...)                 \
    do {                                      \
        if (!(cond)) {                        \
            hb_set_error(__VA_ARGS__);        \
            return 1;                         \
        }                                     \
    } while (0)

#define HB_CHECK_LAUNCH(name)                                              \
    do {                                                                   \
        hipError_t e_ = hipGetLastError();                                 \
        if (e_ != hipSuccess) {                                            \
            hb_set_error("%s: launch failed: %s", name, hipGetErrorString(e_)); \
            return 2;                                                      \
        }                                                                  \
    } while (0)
