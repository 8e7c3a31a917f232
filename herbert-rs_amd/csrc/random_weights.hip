// Seeded random weights from a counter: element i of a tensor is a function of (key, i) alone, the
// same function on the GPU (a kernel) and on the host (threads), so that a model drawn on the GPU and
// a model folder written by the host hold the same bits for the same seed. The reference has no
// random weights (its loader reads checkpoints: crates/backends/backend_common/src/loader_common.rs:1105).
//
// value(key, i) = offset + scale * (b0 + ... + b7 - 1020), b0..b7 the bytes of splitmix64(key, i):
//   z = key + (i + 1) * 0x9E3779B97F4A7C15;  z = (z ^ z >> 30) * 0xBF58476D1CE4E5B9;
//   z = (z ^ z >> 27) * 0x94D049BB133111EB;  z = z ^ z >> 31.
// The sum of eight bytes is near normal (Irwin-Hall: standard deviation sqrt(8 (256^2 - 1) / 12) =
// 209.0227, excess kurtosis -0.15, nothing beyond 4.88 deviations). Only integers are summed; the
// one product and the one sum in float32 are each rounded once (no fused multiply-add), and the
// result is stored as float32 or rounded to bfloat16 (nearest, ties to even).
#include "common.h"
#include <thread>
#include <vector>

HB_MODULE_ERROR_SLOT()

__host__ __device__ inline int random_byte_sum(uint64_t key, uint64_t i) {
    uint64_t z = key + (i + 1) * 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z = z ^ (z >> 31);
    const uint64_t m = 0x00FF00FF00FF00FFull;
    const uint64_t pairs = (z & m) + ((z >> 8) & m);              // four sums of two bytes
    return (int)((pairs * 0x0001000100010001ull) >> 48) - 1020;   // their sum, centred
}

__host__ __device__ inline float random_value(uint64_t key, uint64_t i, float scale, float offset) {
#pragma clang fp contract(off)
    const float scaled = (float)random_byte_sum(key, i) * scale;
    return offset + scaled;
}

__host__ __device__ inline uint16_t bf16_bits_of(float v) {
    union {
        float f;
        uint32_t u;
    } c;
    c.f = v;
    uint32_t u = c.u;
    const uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return (uint16_t)(u >> 16);
}

template <bool BF16>
__global__ void random_fill_kernel(void* out, size_t n, uint64_t key, uint64_t first, float scale, float offset) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float v = random_value(key, first + i, scale, offset);
    if (BF16)
        ((uint16_t*)out)[i] = bf16_bits_of(v);
    else
        ((float*)out)[i] = v;
}

// out[i] = value(key, first + i) for i < n, on the GPU. dtype: HB_F32 or HB_BF16.
extern "C" int hb_random_fill(void* out, int dtype, size_t n, uint64_t key, uint64_t first, float scale, float offset,
                              hipStream_t stream) {
    HB_REQUIRE(dtype == HB_F32 || dtype == HB_BF16, "random_fill: dtype code %d", dtype);
    HB_REQUIRE(out != nullptr || n == 0, "random_fill: no output");
    if (n == 0) return 0;
    const size_t blocks = (n + 255) / 256;
    HB_REQUIRE(blocks <= 0x7fffffffull, "random_fill: %zu elements are more than one launch takes", n);
    if (dtype == HB_BF16)
        random_fill_kernel<true><<<(unsigned)blocks, 256, 0, stream>>>(out, n, key, first, scale, offset);
    else
        random_fill_kernel<false><<<(unsigned)blocks, 256, 0, stream>>>(out, n, key, first, scale, offset);
    HB_CHECK_LAUNCH("random_fill");
    return 0;
}

// The same values into host memory, by up to `threads` threads (no GPU is touched).
extern "C" int hb_random_fill_host(void* out, int dtype, size_t n, uint64_t key, uint64_t first, float scale,
                                   float offset, int threads) {
    HB_REQUIRE(dtype == HB_F32 || dtype == HB_BF16, "random_fill: dtype code %d", dtype);
    HB_REQUIRE(out != nullptr || n == 0, "random_fill: no output");
    if (n == 0) return 0;
    const size_t least = 1 << 16;           // elements that make a thread worth starting
    size_t workers = threads < 1 ? 1 : (size_t)threads;
    if (workers > (n + least - 1) / least) workers = (n + least - 1) / least;
    const size_t per = (n + workers - 1) / workers;
    auto work = [=](size_t a, size_t b) {
        if (dtype == HB_BF16) {
            uint16_t* o = (uint16_t*)out;
            for (size_t i = a; i < b; ++i) o[i] = bf16_bits_of(random_value(key, first + i, scale, offset));
        } else {
            float* o = (float*)out;
            for (size_t i = a; i < b; ++i) o[i] = random_value(key, first + i, scale, offset);
        }
    };
    std::vector<std::thread> pool;
    for (size_t w = 1; w < workers; ++w) pool.emplace_back(work, w * per, (w + 1) * per < n ? (w + 1) * per : n);
    work(0, per < n ? per : n);
    for (auto& t : pool) t.join();
    return 0;
}
