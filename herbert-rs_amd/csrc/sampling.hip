// Choosing the next token on the GPU: argmax and temperature / top-k / top-p sampling.
// The order of candidates is value descending, index ascending among equals; sums that
// decide a cut or a draw are added one value after the other in that order by one
// thread, so that a seed gives the same token as the step-by-step host formulation.
// In xigh/herbert-rs: crates/core/src/sampler.rs:72-145 (logits / temperature, the top_k largest,
// softmax with the maximum taken off, the shortest prefix by probability whose sum reaches top_p,
// a draw r in [0, 1) against the running sum, the last candidate if none), :244-254 (argmax: the
// first of equals); the random numbers are the host's (xorshift64, :30-34, 50-62). On the GPU there:
// crates/backends/backend_metal/shaders/argmax.metal:14-149 (two stages, strict >).
#include "common.h"
#include "noalloc.h"
#include <math.h>
#include <mutex>

HB_MODULE_ERROR_SLOT()

// ------------------------------------------------------------------ argmax
// First index of the largest value of each row (strict > while scanning upwards).
// A row is cut into gridDim.y stretches; each block reduces one stretch to (value, index);
// with more than one stretch a second launch reduces those.
__device__ __forceinline__ bool better(float v, int i, float bv, int bi) {
    return v > bv || (v == bv && i < bi);
}

__global__ void __launch_bounds__(1024)
argmax_kernel(const float* __restrict__ logits, int ld, int V, int* __restrict__ out,
              float* __restrict__ part_v, int* __restrict__ part_i, const float* __restrict__ in_v,
              const int* __restrict__ in_i) {
    __shared__ float best_v[16];
    __shared__ int best_i[16];
    const int r = blockIdx.x;
    const int chunks = gridDim.y;
    const int per = (V + chunks - 1) / chunks;
    const int begin = blockIdx.y * per;
    const int end = begin + per < V ? begin + per : V;
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    if (in_v) {                       // second stage: V candidates (value, index) of this row
        for (int i = threadIdx.x; i < V; i += blockDim.x) {
            const float v = in_v[(size_t)r * V + i];
            const int idx = in_i[(size_t)r * V + i];
            if (better(v, idx, bv, bi)) {
                bv = v;
                bi = idx;
            }
        }
    } else {
        const float* row = logits + (size_t)r * ld;
        bool nan_seen = false;
        for (int i = begin + threadIdx.x; i < end; i += blockDim.x) {
            const float v = row[i];
            nan_seen |= v != v;
            if (v > bv) {
                bv = v;
                bi = i;
            }
        }
        // nothing above -inf, but a NaN: a marker that wins over "nothing at all" among equals
        if (nan_seen && bi == 0x7fffffff) bi = 0x7ffffffe;
    }
#pragma unroll
    for (int off = HB_WAVE / 2; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, HB_WAVE);
        const int oi = __shfl_xor(bi, off, HB_WAVE);
        if (better(ov, oi, bv, bi)) {
            bv = ov;
            bi = oi;
        }
    }
    const int lane = threadIdx.x & (HB_WAVE - 1), wave = threadIdx.x / HB_WAVE;
    if (lane == 0) {
        best_v[wave] = bv;
        best_i[wave] = bi;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        const int nw = (blockDim.x + HB_WAVE - 1) / HB_WAVE;
        for (int w = 1; w < nw; ++w)
            if (better(best_v[w], best_i[w], bv, bi)) {
                bv = best_v[w];
                bi = best_i[w];
            }
        if (part_v) {
            part_v[(size_t)r * chunks + blockIdx.y] = bv;
            part_i[(size_t)r * chunks + blockIdx.y] = bi;
        } else {
            // A row without any value above -inf gives index 0, as a scan from 0 would. If such a row
            // holds a NaN (what a token id out of range leaves of a step: the embedding makes its row
            // NaN) it gives -1, so that the host sees it instead of a token 0 that looks chosen.
            out[r] = bi == 0x7fffffff ? 0 : bi == 0x7ffffffe ? -1 : bi;
        }
    }
}

// scratch_v / scratch_i: [R, chunks] each when chunks > 1 (long rows are cut to fill the GPU).
extern "C" int hb_argmax(const float* logits, int ld, int R, int V, int* out, float* scratch_v,
                         int* scratch_i, int chunks, hipStream_t stream) {
    HB_REQUIRE(R > 0 && V > 0 && ld >= V, "argmax: bad sizes (R=%d, V=%d, ld=%d)", R, V, ld);
    if (chunks <= 1 || !scratch_v || !scratch_i) {
        argmax_kernel<<<dim3(R, 1), 1024, 0, stream>>>(logits, ld, V, out, nullptr, nullptr, nullptr, nullptr);
    } else {
        HB_REQUIRE(chunks <= 1024, "argmax: too many stretches");
        argmax_kernel<<<dim3(R, chunks), 1024, 0, stream>>>(logits, ld, V, out, scratch_v, scratch_i, nullptr,
                                                            nullptr);
        argmax_kernel<<<dim3(R, 1), 64, 0, stream>>>(nullptr, 0, chunks, out, nullptr, nullptr, scratch_v,
                                                     scratch_i);
    }
    HB_CHECK_LAUNCH("argmax");
    return 0;
}

// ---- argmax without a workspace of the caller's (see noalloc.h) ----
// The partial results live in this array: values [MAX_PAIRS] floats, then indices [MAX_PAIRS]
// ints. In host code its name is only a handle for hipGetSymbolAddress: every GPU has a copy
// of its own at an address of its own, looked up once per device and kept below.
static __device__ __align__(256) unsigned char scratch[HB_ARGMAX_NOALLOC_MAX_PAIRS * (sizeof(float) + sizeof(int))];

#define HB_MAX_DEVICES 64
static void* scratch_on_device[HB_MAX_DEVICES] = {nullptr};
static std::mutex scratch_lock;

// The device address of `scratch` on the current device.
static int scratch_address(void** ptr) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    HB_REQUIRE(e == hipSuccess, "argmax (no allocation): hipGetDevice failed: %s", hipGetErrorString(e));
    HB_REQUIRE(dev >= 0 && dev < HB_MAX_DEVICES, "argmax (no allocation): device %d is beyond the %d this library keeps",
               dev, HB_MAX_DEVICES);
    std::lock_guard<std::mutex> guard(scratch_lock);
    if (!scratch_on_device[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        HB_REQUIRE(e == hipSuccess && p, "argmax (no allocation): hipGetSymbolAddress failed on device %d: %s", dev,
                   hipGetErrorString(e));
        scratch_on_device[dev] = p;
    }
    *ptr = scratch_on_device[dev];
    return 0;
}

extern "C" int hb_argmax_noalloc_setup(void) {
    void* p = nullptr;
    return scratch_address(&p);
}

extern "C" int hb_argmax_noalloc(const float* logits, int ld, int R, int V, int* out, hipStream_t stream) {
    HB_REQUIRE(R > 0 && V > 0 && ld >= V, "argmax (no allocation): bad sizes (R=%d, V=%d, ld=%d)", R, V, ld);
    HB_REQUIRE(logits && out, "argmax (no allocation): null logits or out");
    int chunks = V / 8192;
    chunks = chunks > 64 ? 64 : chunks;
    if (chunks <= 1) {
        argmax_kernel<<<dim3(R, 1), 1024, 0, stream>>>(logits, ld, V, out, nullptr, nullptr, nullptr, nullptr);
        HB_CHECK_LAUNCH("argmax (no allocation)");
        return 0;
    }
    HB_REQUIRE((long long)R * chunks <= HB_ARGMAX_NOALLOC_MAX_PAIRS,
               "argmax (no allocation): %d rows x %d stretches = %lld partial results, the library's scratch holds %d; "
               "use hb_argmax with a workspace of your own", R, chunks, (long long)R * chunks,
               HB_ARGMAX_NOALLOC_MAX_PAIRS);
    void* base = nullptr;
    if (scratch_address(&base)) return 1;
    float* part_v = (float*)base;
    int* part_i = (int*)((unsigned char*)base + HB_ARGMAX_NOALLOC_MAX_PAIRS * sizeof(float));
    // every pair the second kernel reads is written by the first: nothing has to be cleared
    argmax_kernel<<<dim3(R, chunks), 1024, 0, stream>>>(logits, ld, V, out, part_v, part_i, nullptr, nullptr);
    argmax_kernel<<<dim3(R, 1), 64, 0, stream>>>(nullptr, 0, chunks, out, nullptr, nullptr, part_v, part_i);
    HB_CHECK_LAUNCH("argmax (no allocation)");
    return 0;
}

// ---------------------------------------------------------------- sampling
// xorshift64 (<<13, >>7, <<17); the draw is the upper 24 bits over 2^24.
__device__ __forceinline__ float xorshift_next_f32(unsigned long long* state) {
    unsigned long long x = *state;
    x ^= x << 13;
    x ^= x >> 7;
    x ^= x << 17;
    *state = x;
    return (float)(x >> 40) / 16777216.0f;
}

// Order-preserving map float -> uint32 (larger float, larger key).
__device__ __forceinline__ uint32_t float_key(float v) {
    const uint32_t u = __float_as_uint(v);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_float(uint32_t k) {
    return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}

#define SAMPLE_THREADS 1024
#define SAMPLE_MAX_K 1024
#define SAMPLE_AHEAD 8           // logits a thread asks for at once when it walks a row
#define SAMPLE_LIST 4096         // keys of one first byte that the kernel keeps in LDS
#define SAMPLE_CHUNK 8192        // logits of a row that one block sifts when a row is shared out over blocks

// (key descending, index ascending) "a before b"
__device__ __forceinline__ bool cand_before(uint32_t ka, int ia, uint32_t kb, int ib) {
    return ka > kb || (ka == kb && ia < ib);
}

__device__ void bitonic_sort_lds(uint32_t* keys, int* idx, int n_pow2) {
    for (int size = 2; size <= n_pow2; size <<= 1) {
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
            __syncthreads();
            for (int i = threadIdx.x; i < n_pow2 / 2; i += blockDim.x) {
                const int lo = 2 * i - (i & (stride - 1));
                const int hi = lo + stride;
                const bool up = (lo & size) == 0;   // this run is sorted "before first"
                const bool hi_first = cand_before(keys[hi], idx[hi], keys[lo], idx[lo]);
                if (hi_first == up) {
                    const uint32_t tk = keys[lo];
                    keys[lo] = keys[hi];
                    keys[hi] = tk;
                    const int ti = idx[lo];
                    idx[lo] = idx[hi];
                    idx[hi] = ti;
                }
            }
        }
    }
    __syncthreads();
}

// The bin of the `remaining`-th largest key, counted from the top of a histogram of 256 bins, by
// the first 256 threads of the block: bin b is it if fewer than `remaining` keys lie above it and
// at least `remaining` in it and above. Writes the chosen bin into the prefix and what is still
// to be found inside that bin. (A single thread walking the bins costs 7 us a byte.)
__device__ __forceinline__ void choose_bin(const int* hist, int* wave_totals, int shift, uint32_t prefix,
                                           int remaining, uint32_t* sel_prefix, int* sel_remaining) {
    const int tid = threadIdx.x, lane = tid & (HB_WAVE - 1);
    int mine = 0, here_and_above = 0;
    if (tid < 256) {
        mine = hist[tid];
        here_and_above = mine;                 // over the lanes from this one up
        for (int d = 1; d < HB_WAVE; d <<= 1) {
            const int other = __shfl_down(here_and_above, d, HB_WAVE);
            if (lane + d < HB_WAVE) here_and_above += other;
        }
        if (lane == 0) wave_totals[tid / HB_WAVE] = here_and_above;
    }
    __syncthreads();
    if (tid < 256) {
        for (int w = tid / HB_WAVE + 1; w < 256 / HB_WAVE; ++w) here_and_above += wave_totals[w];
        const int above = here_and_above - mine;
        if (above < remaining && here_and_above >= remaining) {
            *sel_prefix = prefix | ((uint32_t)tid << shift);
            *sel_remaining = remaining - above;
        }
    }
    __syncthreads();
}

// The largest scaled logit of a chunk of SAMPLE_CHUNK logits (thread t holds elements t, t + 1024, ...
// in v) and the sum of exp(scaled - that), added up in a fixed order: a thread's eight in their
// order, the lanes of a wave by a tree, the waves one after the other. Thread 0 writes both to ms.
__device__ __forceinline__ void chunk_max_and_sum(const float (&v)[SAMPLE_CHUNK / SAMPLE_THREADS], int len,
                                                  float temperature, float* wave_vals, float* ms) {
    constexpr int PER = SAMPLE_CHUNK / SAMPLE_THREADS;
    const int tid = threadIdx.x, lane = tid & (HB_WAVE - 1), wave = tid / HB_WAVE;
    float mv = -INFINITY;
#pragma unroll
    for (int u = 0; u < PER; ++u)
        if (tid + u * SAMPLE_THREADS < len) mv = fmaxf(mv, v[u] / temperature);
    mv = hb_wave_max(mv);
    if (lane == 0) wave_vals[wave] = mv;
    __syncthreads();
    float cmax = wave_vals[0];
    for (int w = 1; w < SAMPLE_THREADS / HB_WAVE; ++w) cmax = fmaxf(cmax, wave_vals[w]);
    __syncthreads();
    float part = 0.f;
    if (cmax != -INFINITY) {
#pragma unroll
        for (int u = 0; u < PER; ++u)
            if (tid + u * SAMPLE_THREADS < len) part += expf(v[u] / temperature - cmax);
    }
    for (int d = HB_WAVE / 2; d > 0; d >>= 1) part += __shfl_down(part, d, HB_WAVE);
    if (lane == 0) wave_vals[wave] = part;
    __syncthreads();
    if (tid == 0) {
        float sum = 0.f;
        for (int w = 0; w < SAMPLE_THREADS / HB_WAVE; ++w) sum += wave_vals[w];
        ms[0] = cmax;
        ms[1] = sum;
    }
}

// The first of two kernels when a row is long: block (chunk, row) keeps the keys of its SAMPLE_CHUNK
// logits in LDS, finds its own top_k among them (ties: lower index first) and leaves them, in any
// order, in pre_key / pre_idx [row][chunk][top_k]. A single block walks a row at about 24 GB/s
// only; shared out over the CUs the 600 KB of a row of 151936 logits are read in a few us.
// chunk_ms != null: it also leaves, in chunk_ms [row][chunk][2], the largest scaled logit of the
// chunk and the sum of exp(scaled - that) over the chunk, added up in a fixed order (a thread's
// eight in their order, the lanes of a wave by a tree, the waves one after the other).
__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_chunk_topk_kernel(const float* __restrict__ logits, int ld, int V, float temperature, int top_k,
                         uint32_t* __restrict__ pre_key, int* __restrict__ pre_idx,
                         float* __restrict__ chunk_ms) {
    __shared__ uint32_t ck[SAMPLE_CHUNK];
    __shared__ float wave_vals[SAMPLE_THREADS / HB_WAVE];
    __shared__ int hist[256];
    __shared__ int wave_counts[SAMPLE_THREADS / HB_WAVE];
    __shared__ uint32_t sel_prefix;
    __shared__ int sel_remaining, n_out, eq_taken;
    const int tid = threadIdx.x, lane = tid & (HB_WAVE - 1), wave = tid / HB_WAVE;
    const int c = blockIdx.x, first = c * SAMPLE_CHUNK;
    const int len = V - first < SAMPLE_CHUNK ? V - first : SAMPLE_CHUNK;
    const float* row = logits + (size_t)blockIdx.y * ld + first;
    const size_t base = ((size_t)blockIdx.y * gridDim.x + c) * top_k;
    constexpr int PER = SAMPLE_CHUNK / SAMPLE_THREADS;
    float v[PER];
#pragma unroll
    for (int u = 0; u < PER; ++u) {
        const int j = tid + u * SAMPLE_THREADS;
        v[u] = j < len ? row[j] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < PER; ++u) {
        const int j = tid + u * SAMPLE_THREADS;
        if (j < len) ck[j] = float_key(v[u] / temperature);
    }
    if (tid == 0) {
        sel_prefix = 0;
        sel_remaining = top_k;
        n_out = 0;
        eq_taken = 0;
    }
    if (chunk_ms)
        chunk_max_and_sum(v, len, temperature, wave_vals, chunk_ms + ((size_t)blockIdx.y * gridDim.x + c) * 2);
    __syncthreads();
    if (len <= top_k) {                       // all of a short chunk
        for (int j = tid; j < len; j += SAMPLE_THREADS) {
            pre_key[base + j] = ck[j];
            pre_idx[base + j] = first + j;
        }
        return;
    }
    for (int shift = 24; shift >= 0; shift -= 8) {
        if (tid < 256) hist[tid] = 0;
        __syncthreads();
        const uint32_t prefix = sel_prefix;
        const int remaining = sel_remaining;
        const uint32_t mask = shift == 24 ? 0u : (0xffffffffu << (shift + 8));
        int run_bin = -1, run = 0;
        for (int j = tid; j < len; j += SAMPLE_THREADS) {
            const uint32_t k = ck[j];
            if ((k & mask) != prefix) continue;
            const int bin = (k >> shift) & 0xff;
            if (bin == run_bin) {
                ++run;
            } else {
                if (run) atomicAdd(&hist[run_bin], run);
                run_bin = bin;
                run = 1;
            }
        }
        if (run) atomicAdd(&hist[run_bin], run);
        __syncthreads();
        choose_bin(hist, wave_counts, shift, prefix, remaining, &sel_prefix, &sel_remaining);
    }
    const uint32_t kth = sel_prefix;
    const int need_eq = sel_remaining;
    // the keys lie in LDS in the order of their indices: the equal ones are ranked stretch by stretch
    for (int start = 0; start < len; start += SAMPLE_THREADS) {
        const int j = start + tid;
        const uint32_t k = j < len ? ck[j] : 0u;
        const bool above = j < len && k > kth, equal = j < len && k == kth;
        const unsigned long long bal = __ballot(equal);
        const int before_lane = __popcll(bal & ((1ull << lane) - 1ull));
        if (lane == 0) wave_counts[wave] = __popcll(bal);
        __syncthreads();
        int before = eq_taken;
        for (int w = 0; w < wave; ++w) before += wave_counts[w];
        if (above || (equal && before + before_lane < need_eq)) {
            const int at = atomicAdd(&n_out, 1);
            pre_key[base + at] = k;
            pre_idx[base + at] = first + j;
        }
        __syncthreads();
        if (tid == 0) {
            int total = 0;
            for (int w = 0; w < SAMPLE_THREADS / HB_WAVE; ++w) total += wave_counts[w];
            eq_taken += total;
        }
        __syncthreads();
    }
}

// One block per row, 0 < top_k <= SAMPLE_MAX_K and top_k < V.
//  1. scaled = logit / temperature; the top_k largest (ties: lower index first) by a
//     radix select over the keys, gathered and sorted in LDS;
//  2. softmax over them; 3. top-p cut and renormalisation; 4. the draw.
// pre_key != null: the row was cut into chunks of SAMPLE_CHUNK logits and sample_chunk_topk_kernel
// has left the top_k of each chunk in pre_key / pre_idx [row][chunk][top_k] (a chunk shorter than
// top_k: all of it); the top_k of the row are among them, and only they are walked.
__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_topk_kernel(const float* __restrict__ logits, int ld, int V, float temperature, int top_k,
                   float top_p, unsigned long long* __restrict__ rng, const int* __restrict__ rng_index,
                   int* __restrict__ out, const uint32_t* __restrict__ pre_key, const int* __restrict__ pre_idx,
                   const float* __restrict__ chunk_ms) {
    __shared__ uint32_t keys[SAMPLE_MAX_K];
    __shared__ int idx[SAMPLE_MAX_K];
    __shared__ float prob[SAMPLE_MAX_K];
    __shared__ int hist[256];
    __shared__ int wave_counts[SAMPLE_THREADS / HB_WAVE];
    __shared__ uint32_t sel_prefix;
    __shared__ int sel_remaining;
    __shared__ int n_gathered;
    __shared__ int eq_taken;

    const float* row = logits + (size_t)blockIdx.x * ld;
    const int tid = threadIdx.x;

    // ---- radix select: the key of the top_k-th largest scaled logit.
    // One block reads a row at about 24 GB/s, so what counts is how often the row is walked:
    // once for the histogram of the keys' first byte (sign and exponent), once more to collect
    // what lies in the chosen bin into LDS (everything above it belongs to the top k anyway);
    // the other three bytes are then decided on that list. A list that does not fit (flat
    // logits) sends the kernel back to walking the row for every byte.
    __shared__ uint32_t cand_key[SAMPLE_LIST];
    __shared__ int cand_idx[SAMPLE_LIST];
    __shared__ int eq_idx[SAMPLE_MAX_K];
    __shared__ int cand_count, eq_count;
    const int lane = tid & (HB_WAVE - 1), wave = tid / HB_WAVE;
    // f(key, index) for every element of the row, SAMPLE_AHEAD loads of a thread in flight at once
    const int chunks = (V + SAMPLE_CHUNK - 1) / SAMPLE_CHUNK;
    auto walk_row = [&](auto&& f) {
        if (pre_key) {
            const size_t first = (size_t)blockIdx.x * chunks * top_k;
            for (int t = tid; t < chunks * top_k; t += SAMPLE_THREADS) {
                const int c = t / top_k, j = t - c * top_k;
                const int len = V - c * SAMPLE_CHUNK < SAMPLE_CHUNK ? V - c * SAMPLE_CHUNK : SAMPLE_CHUNK;
                if (j < (len < top_k ? len : top_k)) f(pre_key[first + t], pre_idx[first + t]);
            }
            return;
        }
        for (int base = tid; base < V; base += SAMPLE_AHEAD * SAMPLE_THREADS) {
            float v[SAMPLE_AHEAD];
#pragma unroll
            for (int u = 0; u < SAMPLE_AHEAD; ++u) {
                const int i = base + u * SAMPLE_THREADS;
                v[u] = i < V ? row[i] : 0.f;
            }
#pragma unroll
            for (int u = 0; u < SAMPLE_AHEAD; ++u) {
                const int i = base + u * SAMPLE_THREADS;
                if (i < V) f(float_key(v[u] / temperature), i);
            }
        }
    };
    // counts the byte at `shift` of the keys that f hands to count(key), runs of one bin at a time
    auto choose_byte = [&](int shift, auto&& walk) {
        if (tid < 256) hist[tid] = 0;
        __syncthreads();
        const uint32_t prefix = sel_prefix;
        const int remaining = sel_remaining;
        const uint32_t mask = shift == 24 ? 0u : (0xffffffffu << (shift + 8));
        int run_bin = -1, run = 0;
        walk([&](uint32_t k, int) {
            if ((k & mask) != prefix) return;
            const int bin = (k >> shift) & 0xff;
            if (bin == run_bin) {
                ++run;
            } else {
                if (run) atomicAdd(&hist[run_bin], run);
                run_bin = bin;
                run = 1;
            }
        });
        if (run) atomicAdd(&hist[run_bin], run);
        __syncthreads();
        choose_bin(hist, wave_counts, shift, prefix, remaining, &sel_prefix, &sel_remaining);
    };
    if (tid == 0) {
        sel_prefix = 0;
        sel_remaining = top_k;
        n_gathered = 0;
        eq_taken = 0;
        eq_count = 0;
        cand_count = 0;
    }
    choose_byte(24, walk_row);
    {
        const uint32_t first = sel_prefix >> 24;
        walk_row([&](uint32_t k, int i) {
            const uint32_t byte = k >> 24;
            if (byte > first) {                       // above the chosen bin: one of the top k
                const int at = atomicAdd(&n_gathered, 1);
                keys[at] = k;
                idx[at] = i;
            } else if (byte == first) {
                const int at = atomicAdd(&cand_count, 1);
                if (at < SAMPLE_LIST) {
                    cand_key[at] = k;
                    cand_idx[at] = i;
                }
            }
        });
    }
    __syncthreads();
    const int listed = cand_count;
    const bool from_list = listed <= SAMPLE_LIST;
    auto walk_list = [&](auto&& f) {
        for (int c = tid; c < listed; c += SAMPLE_THREADS) f(cand_key[c], cand_idx[c]);
    };
    for (int shift = 16; shift >= 0; shift -= 8) {
        if (from_list) choose_byte(shift, walk_list);
        else choose_byte(shift, walk_row);
    }
    const uint32_t kth = sel_prefix;        // key of the k-th largest
    const int need_eq = sel_remaining;      // how many of the equal keys belong to the top k

    // ---- gather: the keys above kth in any order (the sort that follows orders them), and of the
    // equal ones the need_eq with the lowest indices. The equal ones are listed first; only a
    // list that overflows is walked in index order.
    auto take = [&](uint32_t k, int i) {
        if (k > kth) {
            if (from_list && (k >> 24) > (kth >> 24)) return;      // gathered before
            const int at = atomicAdd(&n_gathered, 1);
            keys[at] = k;
            idx[at] = i;
        } else if (k == kth) {
            const int e = atomicAdd(&eq_count, 1);
            if (e < SAMPLE_MAX_K) eq_idx[e] = i;
        }
    };
    if (from_list) {
        walk_list(take);
    } else {
        __syncthreads();
        if (tid == 0) n_gathered = 0;                  // (what the first walk gathered is gathered again)
        __syncthreads();
        walk_row(take);
    }
    __syncthreads();
    const int total_eq = eq_count;
    if (total_eq <= SAMPLE_MAX_K) {
        // rank of an equal key = how many of the listed ones have a lower index
        for (int e = tid; e < total_eq; e += blockDim.x) {
            const int mine = eq_idx[e];
            int rank = 0;
            if (total_eq > need_eq)
                for (int o = 0; o < total_eq; ++o) rank += eq_idx[o] < mine;
            if (rank < need_eq) {
                const int at = atomicAdd(&n_gathered, 1);
                keys[at] = kth;
                idx[at] = mine;
            }
        }
        __syncthreads();
    } else {
        for (int base = 0; base < V; base += blockDim.x) {
            const int i = base + tid;
            const bool equal = i < V && float_key(row[i] / temperature) == kth;
            // ordered rank of the equal ones within this stretch of the row
            const unsigned long long bal = __ballot(equal);
            const int before_lane = __popcll(bal & ((1ull << lane) - 1ull));
            if (lane == 0) wave_counts[wave] = __popcll(bal);
            __syncthreads();
            int before = eq_taken;
            for (int w = 0; w < wave; ++w) before += wave_counts[w];
            const int rank = before + before_lane;
            if (equal && rank < need_eq) {
                const int at = atomicAdd(&n_gathered, 1);
                keys[at] = kth;
                idx[at] = i;
            }
            __syncthreads();
            if (tid == 0) {
                int total = 0;
                for (int w = 0; w < SAMPLE_THREADS / HB_WAVE; ++w) total += wave_counts[w];
                eq_taken += total;
            }
            __syncthreads();
        }
    }
    const int n = n_gathered;   // == top_k
    int n_pow2 = 1;
    while (n_pow2 < n) n_pow2 <<= 1;
    for (int i = n + tid; i < n_pow2; i += blockDim.x) {
        keys[i] = 0u;
        idx[i] = 0x7fffffff;
    }
    bitonic_sort_lds(keys, idx, n_pow2);

    // ---- softmax in candidate order (the first candidate holds the maximum)
    const float max_val = key_float(keys[0]);
    for (int i = tid; i < n; i += blockDim.x) prob[i] = expf(key_float(keys[i]) - max_val);
    __syncthreads();
    __shared__ float inv_sum_s;
    if (tid == 0) {
        float sum = 0.f;
        if (chunk_ms) {
            // every logit of the row counts in the softmax: the chunks' sums, in the order of the chunks
            const float* ms = chunk_ms + (size_t)blockIdx.x * chunks * 2;
            for (int c = 0; c < chunks; ++c)
                if (ms[2 * c] != -INFINITY) sum += ms[2 * c + 1] * expf(ms[2 * c] - max_val);
        } else {
            for (int i = 0; i < n; ++i) sum += prob[i];
        }
        inv_sum_s = 1.0f / sum;
    }
    __syncthreads();
    for (int i = tid; i < n; i += blockDim.x) prob[i] *= inv_sum_s;
    __syncthreads();

    __shared__ int n_kept;
    if (tid == 0) n_kept = n;
    if (top_p < 1.0f) {
        // order by probability descending (index ascending among equals); exp can map two
        // different keys to one probability, so this is a sort of its own
        for (int i = tid; i < n_pow2; i += blockDim.x) keys[i] = i < n ? float_key(prob[i]) : 0u;
        bitonic_sort_lds(keys, idx, n_pow2);
        for (int i = tid; i < n; i += blockDim.x) prob[i] = key_float(keys[i]);
        __syncthreads();
        if (tid == 0) {
            float cum = 0.f;
            int cutoff = n;
            for (int i = 0; i < n; ++i) {
                cum += prob[i];
                if (cum >= top_p) {
                    cutoff = i + 1;
                    break;
                }
            }
            float sum = 0.f;
            for (int i = 0; i < cutoff; ++i) sum += prob[i];
            inv_sum_s = 1.0f / sum;
            n_kept = cutoff;
            // The candidates are the largest of a longer row: the prefix is the row's own only if
            // the sum has reached top_p and everything kept is more probable than the last
            // candidate (what was left out is at most as probable as that one, and among equals
            // the index decides).
            if (chunk_ms && !(cum >= top_p && prob[cutoff - 1] > prob[n - 1])) n_kept = -1;
        }
        __syncthreads();
        const int kept = n_kept;
        for (int i = tid; i < kept; i += blockDim.x) prob[i] *= inv_sum_s;
    }
    __syncthreads();
    if (n_kept < 0) {                 // undecided: no draw is taken, the caller sees -1
        if (tid == 0) out[blockIdx.x] = -1;
        return;
    }

    if (tid == 0) {
        unsigned long long* st = rng + (rng_index ? rng_index[blockIdx.x] : blockIdx.x);
        const float r = xorshift_next_f32(st);
        const int kept = n_kept;
        float cum = 0.f;
        int chosen = idx[kept - 1];
        for (int i = 0; i < kept; ++i) {
            cum += prob[i];
            if (r < cum) {
                chosen = idx[i];
                break;
            }
        }
        out[blockIdx.x] = chosen;
    }
}

// ---- the general path: candidates of a row in global scratch as (key, index) pairs.
// prepare: pairs[r, i] = (key(logit / temperature), i) for i < V, padding up to P2 (a power
// of two) with (0, INT_MAX), which sorts last.
__global__ void sample_prepare_kernel(const float* __restrict__ logits, int ld, int V, int P2,
                                      float temperature, uint32_t* __restrict__ keys,
                                      int* __restrict__ idx) {
    const int r = blockIdx.y;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= P2) return;
    const size_t o = (size_t)r * P2 + i;
    if (i < V) {
        keys[o] = float_key(logits[(size_t)r * ld + i] / temperature);
        idx[o] = i;
    } else {
        keys[o] = 0u;
        idx[o] = 0x7fffffff;
    }
}

// One compare-exchange stage of a bitonic sort over every row.
__global__ void sample_bitonic_stage_kernel(uint32_t* __restrict__ keys, int* __restrict__ idx, int P2,
                                            int size, int stride) {
    const int r = blockIdx.y;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= P2 / 2) return;
    uint32_t* k = keys + (size_t)r * P2;
    int* x = idx + (size_t)r * P2;
    const int lo = 2 * i - (i & (stride - 1));
    const int hi = lo + stride;
    const bool up = (lo & size) == 0;
    const bool hi_first = cand_before(k[hi], x[hi], k[lo], x[lo]);
    if (hi_first == up) {
        const uint32_t tk = k[lo];
        k[lo] = k[hi];
        k[hi] = tk;
        const int ti = x[lo];
        x[lo] = x[hi];
        x[hi] = ti;
    }
}

// The stages of a bitonic sort whose stride is below SORT_BLOCK / 2, on one stretch of SORT_BLOCK
// elements in LDS: every step from first_size up to last_size, and within the first one only the
// strides from first_stride down (the larger ones were done in global memory). With first_size = 2
// and last_size = SORT_BLOCK this sorts the stretch from scratch.
#define SORT_BLOCK 4096
__global__ void __launch_bounds__(1024)
sample_bitonic_local_kernel(uint32_t* __restrict__ keys, int* __restrict__ idx, int P2, int first_size,
                            int last_size, int first_stride) {
    __shared__ uint32_t lk[SORT_BLOCK];
    __shared__ int lx[SORT_BLOCK];
    const int block = P2 < SORT_BLOCK ? P2 : SORT_BLOCK;
    const size_t base = (size_t)blockIdx.y * P2 + (size_t)blockIdx.x * block;
    for (int i = threadIdx.x; i < block; i += blockDim.x) {
        lk[i] = keys[base + i];
        lx[i] = idx[base + i];
    }
    const int offset = blockIdx.x * block;          // position of this stretch in its row: decides the direction
    for (int size = first_size; size <= last_size; size <<= 1) {
        for (int stride = size == first_size ? first_stride : size >> 1; stride > 0; stride >>= 1) {
            __syncthreads();
            for (int i = threadIdx.x; i < block / 2; i += blockDim.x) {
                const int lo = 2 * i - (i & (stride - 1));
                const int hi = lo + stride;
                const bool up = ((offset + lo) & size) == 0;
                const bool hi_first = cand_before(lk[hi], lx[hi], lk[lo], lx[lo]);
                if (hi_first == up) {
                    const uint32_t tk = lk[lo];
                    lk[lo] = lk[hi];
                    lk[hi] = tk;
                    const int ti = lx[lo];
                    lx[lo] = lx[hi];
                    lx[hi] = ti;
                }
            }
        }
    }
    __syncthreads();
    for (int i = threadIdx.x; i < block; i += blockDim.x) {
        keys[base + i] = lk[i];
        idx[base + i] = lx[i];
    }
}

// finish: one block per row over its first n candidates (sorted when sorted != 0, else in index
// order). The sums that decide a cut or a draw run over the candidates in their order, a stretch
// of FINISH_CHUNK at a time: a thread adds up four neighbours, the threads' sums are scanned in
// a fixed order (within a wave, then over the waves), and the thread in whose four the sum first
// passes the mark walks them one by one. The order of additions is fixed; it is not the order of
// a single running sum, whose rounding may put a draw that falls within an ulp of a boundary on
// the other side of it.
#define FINISH_CHUNK 4096
// Adds value(i) for i in [0, n) in order. MARK 0: no mark; 1: stops at the first i whose running
// sum is >= mark; 2: at the first whose running sum is > mark. Returns the sum over all (MARK 0)
// or up to and including the marked one; *marked = its i, or -1.
template <int MARK, class Value>
__device__ float ordered_sum(int n, float mark, int* marked, float* buf, float* wave_totals, int* s_found,
                             float* s_total, Value&& value) {
    const int tid = threadIdx.x, lane = tid & (HB_WAVE - 1), wave = tid / HB_WAVE;
    const int waves = blockDim.x / HB_WAVE;
    float carry = 0.f;
    __syncthreads();                       // nobody is still reading what an earlier call found
    if (tid == 0) *s_found = -1;
    for (int c = 0; c < n; c += FINISH_CHUNK) {
        const int m = n - c < FINISH_CHUNK ? n - c : FINISH_CHUNK;
        __syncthreads();
        for (int i = tid; i < m; i += blockDim.x) buf[i] = value(c + i);
        __syncthreads();
        float part = 0.f;
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (4 * tid + e < m) part += buf[4 * tid + e];
        float incl = part;                                   // over the threads of this wave up to this one
        for (int d = 1; d < HB_WAVE; d <<= 1) {
            const float other = __shfl_up(incl, d, HB_WAVE);
            if (lane >= d) incl += other;
        }
        float excl = __shfl_up(incl, 1, HB_WAVE);            // the lane before: its sum is where this one starts
        if (lane == 0) excl = 0.f;
        if (lane == HB_WAVE - 1) wave_totals[wave] = incl;
        __syncthreads();
        float before = carry;                                // everything before this wave
        for (int w = 0; w < wave; ++w) before += wave_totals[w];
        float chunk_total = 0.f;
        for (int w = 0; w < waves; ++w) chunk_total += wave_totals[w];
        if (MARK) {
            const float upto = before + incl, until = before + excl;    // with and without this thread's four
            const bool passes = MARK == 1 ? upto >= mark : upto > mark;
            const bool passed = MARK == 1 ? until >= mark : until > mark;
            if (passes && !passed && 4 * tid < m) {
                // the first thread whose sum passes the mark: the scan is monotonic, so there is one
                float cum = until;
                int at = 4 * tid;
                for (int e = 0; e < 4 && 4 * tid + e < m; ++e) {
                    cum += buf[4 * tid + e];
                    at = 4 * tid + e;
                    if (MARK == 1 ? cum >= mark : cum > mark) break;
                }
                *s_found = c + at;
                *s_total = cum;
            }
            __syncthreads();
            if (*s_found >= 0) {
                *marked = *s_found;
                return *s_total;
            }
        }
        carry += chunk_total;
    }
    if (MARK) *marked = -1;
    return carry;
}

__global__ void __launch_bounds__(1024)
sample_finish_kernel(const uint32_t* __restrict__ keys, const int* __restrict__ idx, int P2, int n,
                     int sorted, float top_p, unsigned long long* __restrict__ rng,
                     const int* __restrict__ rng_index, int* __restrict__ out) {
    __shared__ float buf[FINISH_CHUNK];
    __shared__ float red[16];
    __shared__ float s_max, s_r, s_total;
    __shared__ int s_found;
    const uint32_t* k = keys + (size_t)blockIdx.x * P2;
    const int* x = idx + (size_t)blockIdx.x * P2;
    const int tid = threadIdx.x;

    // maximum: the first candidate when sorted, else a reduction (its order does not matter)
    if (sorted) {
        if (tid == 0) s_max = key_float(k[0]);
    } else {
        float mv = -INFINITY;
        for (int i = tid; i < n; i += blockDim.x) mv = fmaxf(mv, key_float(k[i]));
        mv = hb_wave_max(mv);
        if ((tid & (HB_WAVE - 1)) == 0) red[tid / HB_WAVE] = mv;
        __syncthreads();
        if (tid == 0) {
            for (int w = 1; w < (int)(blockDim.x / HB_WAVE); ++w) mv = fmaxf(mv, red[w]);
            s_max = mv;
        }
    }
    if (tid == 0) {
        unsigned long long* st = rng + (rng_index ? rng_index[blockIdx.x] : blockIdx.x);
        s_r = xorshift_next_f32(st);
    }
    __syncthreads();
    const float max_val = s_max, r = s_r;
    int marked;

    // the softmax denominator
    const float inv = 1.0f / ordered_sum<0>(n, 0.f, &marked, buf, red, &s_found, &s_total,
                                            [&](int i) { return expf(key_float(k[i]) - max_val); });
    // the top-p cut (candidates are sorted then) and the sum of the kept ones
    int kept = n;
    float inv2 = 1.0f;
    if (top_p < 1.0f) {
        const float sum2 = ordered_sum<1>(n, top_p, &marked, buf, red, &s_found, &s_total,
                                          [&](int i) { return expf(key_float(k[i]) - max_val) * inv; });
        if (marked >= 0) kept = marked + 1;
        inv2 = 1.0f / sum2;
    }
    // the draw: the first candidate whose running probability exceeds r, else the last one kept
    const bool renorm = top_p < 1.0f;
    ordered_sum<2>(kept, r, &marked, buf, red, &s_found, &s_total, [&](int i) {
        const float p = expf(key_float(k[i]) - max_val) * inv;
        return renorm ? p * inv2 : p;
    });
    if (tid == 0) out[blockIdx.x] = x[marked >= 0 ? marked : kept - 1];
}

// Sample one token per row. temperature > 0. top_k == 0 means no top-k; top_p >= 1 none.
// scratch_keys / scratch_idx: [R, P2] each, P2 = the power of two >= V, used by the general
// path only (top_k == 0, top_k >= V or top_k > 1024).
// pre_key / pre_idx: [R, ceil(V / 8192), top_k] each, optional: with them a long row (more than two
// chunks of 8192) is first sifted by a block a chunk.
extern "C" int hb_sample(const float* logits, int ld, int R, int V, float temperature, int top_k,
                         float top_p, unsigned long long* rng, const int* rng_index, int* out,
                         uint32_t* scratch_keys, int* scratch_idx, int P2, uint32_t* pre_key, int* pre_idx,
                         hipStream_t stream) {
    HB_REQUIRE(R > 0 && V > 0 && ld >= V, "sample: bad sizes (R=%d, V=%d, ld=%d)", R, V, ld);
    HB_REQUIRE(temperature > 0.f, "sample: temperature must be > 0 (0 is argmax)");
    HB_REQUIRE(top_k >= 0, "sample: top_k must be >= 0");
    const bool k_active = top_k > 0 && top_k < V;
    if (k_active && top_k <= SAMPLE_MAX_K) {
        const int chunks = (V + SAMPLE_CHUNK - 1) / SAMPLE_CHUNK;
        const bool sift = pre_key && pre_idx && chunks > 2 && R <= 65535;
        if (sift) {
            sample_chunk_topk_kernel<<<dim3(chunks, R), SAMPLE_THREADS, 0, stream>>>(logits, ld, V, temperature,
                                                                                    top_k, pre_key, pre_idx, nullptr);
            HB_CHECK_LAUNCH("sample_chunk_topk");
        }
        sample_topk_kernel<<<R, SAMPLE_THREADS, 0, stream>>>(logits, ld, V, temperature, top_k, top_p, rng,
                                                           rng_index, out, sift ? pre_key : nullptr,
                                                           sift ? pre_idx : nullptr, nullptr);
        HB_CHECK_LAUNCH("sample_topk");
        return 0;
    }
    HB_REQUIRE(scratch_keys && scratch_idx, "sample: this top_k needs the scratch buffers");
    HB_REQUIRE(P2 >= V && (P2 & (P2 - 1)) == 0, "sample: scratch width %d is no power of two >= %d", P2,
               V);
    dim3 pgrid((P2 + 255) / 256, R);
    sample_prepare_kernel<<<pgrid, 256, 0, stream>>>(logits, ld, V, P2, temperature, scratch_keys,
                                                     scratch_idx);
    HB_CHECK_LAUNCH("sample_prepare");
    const int sorted = (k_active || top_p < 1.0f) ? 1 : 0;
    if (sorted) {
        // stretches of SORT_BLOCK are sorted in LDS; a larger step does its wide strides in global
        // memory, one kernel each, and the rest again in LDS
        const int block = P2 < SORT_BLOCK ? P2 : SORT_BLOCK;
        dim3 lgrid(P2 / block, R), sgrid((P2 / 2 + 255) / 256, R);
        sample_bitonic_local_kernel<<<lgrid, 1024, 0, stream>>>(scratch_keys, scratch_idx, P2, 2, block, 1);
        for (int size = 2 * block; size <= P2; size <<= 1) {
            for (int stride = size >> 1; stride >= block; stride >>= 1)
                sample_bitonic_stage_kernel<<<sgrid, 256, 0, stream>>>(scratch_keys, scratch_idx, P2, size,
                                                                       stride);
            sample_bitonic_local_kernel<<<lgrid, 1024, 0, stream>>>(scratch_keys, scratch_idx, P2, size, size,
                                                                    block / 2);
        }
        HB_CHECK_LAUNCH("sample_sort");
    }
    const int n = k_active ? top_k : V;
    sample_finish_kernel<<<R, 1024, 0, stream>>>(scratch_keys, scratch_idx, P2, n, sorted, top_p, rng,
                                                 rng_index, out);
    HB_CHECK_LAUNCH("sample_finish");
    return 0;
}

// Temperature sampling over a whole long row (no top-k, no top-p), in two kernels: a block for every
// SAMPLE_CHUNK logits leaves the chunk's largest scaled logit and its sum of exponentials; a block a
// row then adds up the chunks in their order for the softmax's denominator, takes the draw, finds
// the chunk in which the running probability passes it and walks that chunk (ordered_sum). The
// candidates stay in index order, as the reference has them here (crates/core/src/sampler.rs:84-144).
__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_chunk_sums_kernel(const float* __restrict__ logits, int ld, int V, float temperature,
                         float* __restrict__ chunk_ms) {
    __shared__ float wave_vals[SAMPLE_THREADS / HB_WAVE];
    constexpr int PER = SAMPLE_CHUNK / SAMPLE_THREADS;
    const int tid = threadIdx.x, c = blockIdx.x, first = c * SAMPLE_CHUNK;
    const int len = V - first < SAMPLE_CHUNK ? V - first : SAMPLE_CHUNK;
    const float* row = logits + (size_t)blockIdx.y * ld + first;
    float v[PER];
#pragma unroll
    for (int u = 0; u < PER; ++u) {
        const int j = tid + u * SAMPLE_THREADS;
        v[u] = j < len ? row[j] : 0.f;
    }
    chunk_max_and_sum(v, len, temperature, wave_vals, chunk_ms + ((size_t)blockIdx.y * gridDim.x + c) * 2);
}

__global__ void __launch_bounds__(1024)
sample_all_finish_kernel(const float* __restrict__ logits, int ld, int V, float temperature,
                         const float* __restrict__ chunk_ms, unsigned long long* __restrict__ rng,
                         const int* __restrict__ rng_index, int* __restrict__ out) {
    __shared__ float buf[FINISH_CHUNK];
    __shared__ float red[16];
    __shared__ float s_max, s_inv, s_r, s_before, s_total;
    __shared__ int s_chunk, s_found;
    const int tid = threadIdx.x;
    const int chunks = (V + SAMPLE_CHUNK - 1) / SAMPLE_CHUNK;
    const float* row = logits + (size_t)blockIdx.x * ld;
    if (tid == 0) {
        const float* ms = chunk_ms + (size_t)blockIdx.x * chunks * 2;
        float mx = -INFINITY;
        for (int c = 0; c < chunks; ++c) mx = fmaxf(mx, ms[2 * c]);
        float z = 0.f;
        for (int c = 0; c < chunks; ++c)
            if (ms[2 * c] != -INFINITY) z += ms[2 * c + 1] * expf(ms[2 * c] - mx);
        const float inv = 1.0f / z;
        unsigned long long* st = rng + (rng_index ? rng_index[blockIdx.x] : blockIdx.x);
        const float r = xorshift_next_f32(st);
        // the chunk in which the running probability first exceeds the draw
        float before = 0.f;
        int chosen = -1;
        for (int c = 0; c < chunks; ++c) {
            const float mass = ms[2 * c] != -INFINITY ? ms[2 * c + 1] * expf(ms[2 * c] - mx) * inv : 0.f;
            if (r < before + mass) {
                chosen = c;
                break;
            }
            before += mass;
        }
        s_max = mx;
        s_inv = inv;
        s_r = r;
        s_before = before;
        s_chunk = chosen;
    }
    __syncthreads();
    if (s_chunk < 0) {                      // the draw lies beyond the last running sum: the last token
        if (tid == 0) out[blockIdx.x] = V - 1;
        return;
    }
    const int first = s_chunk * SAMPLE_CHUNK;
    const int len = V - first < SAMPLE_CHUNK ? V - first : SAMPLE_CHUNK;
    const float max_val = s_max, inv = s_inv;
    int marked;
    ordered_sum<2>(len, s_r - s_before, &marked, buf, red, &s_found, &s_total,
                   [&](int i) { return expf(row[first + i] / temperature - max_val) * inv; });
    // (a chunk whose own walk ends just short of the mark, by rounding: its last token)
    if (tid == 0) out[blockIdx.x] = first + (marked >= 0 ? marked : len - 1);
}

// chunk_ms: float [R, ceil(V / 8192), 2].
extern "C" int hb_sample_all(const float* logits, int ld, int R, int V, float temperature, unsigned long long* rng,
                             const int* rng_index, int* out, float* chunk_ms, hipStream_t stream) {
    HB_REQUIRE(R > 0 && R <= 65535 && V > 0 && ld >= V, "sample (whole row): bad sizes (R=%d, V=%d, ld=%d)", R, V, ld);
    HB_REQUIRE(temperature > 0.f, "sample (whole row): temperature must be > 0 (0 is argmax)");
    HB_REQUIRE(chunk_ms, "sample (whole row): needs its buffer");
    const int chunks = (V + SAMPLE_CHUNK - 1) / SAMPLE_CHUNK;
    sample_chunk_sums_kernel<<<dim3(chunks, R), SAMPLE_THREADS, 0, stream>>>(logits, ld, V, temperature, chunk_ms);
    HB_CHECK_LAUNCH("sample_chunk_sums");
    sample_all_finish_kernel<<<R, 1024, 0, stream>>>(logits, ld, V, temperature, chunk_ms, rng, rng_index, out);
    HB_CHECK_LAUNCH("sample_all_finish");
    return 0;
}

// Top-p without top-k on a long row, the quick way: the prefix by descending probability whose
// sum reaches top_p nearly always lies among the SAMPLE_MAX_K largest logits, so only those are
// found and sorted (as for top_k = SAMPLE_MAX_K), while the softmax runs over the whole row (the
// chunks' sums). A row whose prefix does not end inside those candidates gets out[r] = -1 and its
// generator is left as it was: the caller samples that row with hb_sample.
// pre_key / pre_idx: [R, ceil(V / 8192), 1024] each; chunk_ms: float [R, ceil(V / 8192), 2].
extern "C" int hb_sample_nucleus(const float* logits, int ld, int R, int V, float temperature, float top_p,
                                 unsigned long long* rng, const int* rng_index, int* out, uint32_t* pre_key,
                                 int* pre_idx, float* chunk_ms, hipStream_t stream) {
    HB_REQUIRE(R > 0 && R <= 65535 && V > SAMPLE_MAX_K && ld >= V,
               "sample (top-p first): bad sizes (R=%d, V=%d, ld=%d); rows must be longer than %d", R, V, ld,
               SAMPLE_MAX_K);
    HB_REQUIRE(temperature > 0.f && top_p < 1.0f, "sample (top-p first): needs temperature > 0 and top_p < 1");
    HB_REQUIRE(pre_key && pre_idx && chunk_ms, "sample (top-p first): needs its three buffers");
    const int chunks = (V + SAMPLE_CHUNK - 1) / SAMPLE_CHUNK;
    sample_chunk_topk_kernel<<<dim3(chunks, R), SAMPLE_THREADS, 0, stream>>>(logits, ld, V, temperature,
                                                                            SAMPLE_MAX_K, pre_key, pre_idx, chunk_ms);
    HB_CHECK_LAUNCH("sample_chunk_topk (top-p first)");
    sample_topk_kernel<<<R, SAMPLE_THREADS, 0, stream>>>(logits, ld, V, temperature, SAMPLE_MAX_K, top_p, rng,
                                                       rng_index, out, pre_key, pre_idx, chunk_ms);
    HB_CHECK_LAUNCH("sample_topk (top-p first)");
    return 0;
}

// Leaves one token a row to choose from: every other logit of row rows[i] becomes -inf
// (crates/core/src/sampler.rs:234-243 of the reference). rows, tokens: int32 [n], device memory.
__global__ void force_token_kernel(float* __restrict__ logits, int ld, int V, const int* __restrict__ rows,
                                   const int* __restrict__ tokens) {
    const int j = blockIdx.x * blockDim.x + threadIdx.x;
    const int keep = tokens[blockIdx.y];
    if (j < V && j != keep) logits[(size_t)rows[blockIdx.y] * ld + j] = -INFINITY;
}

extern "C" int hb_force_tokens(float* logits, int ld, int R, int V, const int* rows, const int* tokens, int n,
                               hipStream_t stream) {
    HB_REQUIRE(R > 0 && V > 0 && ld >= V && n > 0 && n <= 65535, "force_tokens: bad sizes (R=%d, V=%d, ld=%d, n=%d)",
               R, V, ld, n);
    HB_REQUIRE(rows && tokens, "force_tokens: needs the rows and their tokens");
    force_token_kernel<<<dim3((V + 255) / 256, n), 256, 0, stream>>>(logits, ld, V, rows, tokens);
    HB_CHECK_LAUNCH("force_tokens");
    return 0;
}
