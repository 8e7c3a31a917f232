// bfloat16 matrix products on the gfx950 matrix cores, float32 accumulation:
//   C[m, n] (+)= sum_k X[m, k] * W[n, k]        X [M, K], W [N, K], both k-contiguous
//   few rows (M <= 16, decoding): HBM-bound. The weights stream from memory straight into
//     16x16x32 MFMA operands (each is used once), the waves of a workgroup split K between
//     them and add their parts through LDS in a fixed order.
//   tiled: 32x32x16 MFMA; tiles loaded from global memory straight into rings of LDS stages, a
//     step of 64 k ahead of the MFMAs that consume them; with few tiles K is cut into slices
//     over further workgroups, whose sums a second kernel (or the caller's next kernel) adds up.
//     256 x 256, 256 x 128 or 128 x 128 for prompts; one block of rows high (128 x 32, 128 x 64,
//     256 x 64) for at most 64 rows, where it competes with the few-row kernel (see plan_gemm).
// Between a product that adds to the residual stream and the next one an RMSNorm can be handed
// on instead of run (see NormHandoff).
// In both the weight rows are the MFMA's first operand, so a lane ends up with runs of four
// consecutive n of one m: row-major stores of C are vector stores.
// Epilogues: 0 store float32, 1 add to float32 (the residual stream), 2 SwiGLU to bfloat16
// (weight rows interleaved in blocks of 16: gate rows, then the up rows of the same outputs),
// 3 (tiled, an entry point of its own) the q/k/v projection with per-head norm, rotation and
// cache write.
// In xigh/herbert-rs: crates/backends/backend_bf16/src/kernels.rs:154-164 is the product; the inputs are rounded to
// bfloat16 before they are multiplied, as crates/backends/backend_bf16_avx512/src/avx512_bf16_matvec.S:1-12 does
// (float32 sums); SwiGLU in the epilogue as crates/backends/backend_metal/shaders/fused_gate_up_swiglu.metal:27-83;
// the residual added in the epilogue as the Metal backend's down projection
// (crates/backends/backend_metal/src/backend.rs:488-507); the norm that follows a residual sum prepared with it as
// crates/backends/backend_metal/shaders/rms_norm_residual.metal:31-78 fuses the two.
#include "common.h"
#include <mutex>
#include <unordered_set>

HB_MODULE_ERROR_SLOT()

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

#define EPI_STORE 0
#define EPI_ADD 1
#define EPI_SWIGLU 2
#define EPI_QKV 3

// silu(g) u with the hardware's reciprocal (1 ulp; the result is rounded to bfloat16): a full division
// is a dozen instructions, and the epilogue of a 256 x 256 tile does 128 of these a lane
__device__ __forceinline__ float silu_mul(float g, float u) {
    return g * __builtin_amdgcn_rcpf(1.0f + __expf(-g)) * u;
}

// ---------------------------------------------------------------- few rows
// Workgroup: WAVES waves, NB blocks of 16 weight rows, MB blocks of 16 activation rows (built for
// MB = 1: products of more than 16 rows go to the tiled kernel).
// Wave w takes the k-steps (32 wide) s = w, w + WAVES, ...; it loads U steps ahead of the
// ones it multiplies, so that enough bytes are in flight to keep HBM busy.
// x * g of 8 consecutive k as an MFMA operand; the squares of x are added to ss.
__device__ __forceinline__ bf16x8 normed_operand(const f32x4 xf[2], const f32x4 g[2], float& ss) {
    bf16x8 r;
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float v = xf[h][e];
            ss = fmaf(v, v, ss);
            r[h * 4 + e] = (__bf16)(v * g[h][e]);
        }
    return r;
}

// NORM: the activations are the float32 residual stream and the product is RMSNorm(x) W^T:
//   y = (x * inv * g) W^T = inv * ((x * g) W^T),  inv = 1 / sqrt(mean(x^2) + eps) per row,
// so x * g goes through the matrix cores (rounded to bfloat16) and inv scales the sums at the
// end; the sum of squares comes from the values the lanes load anyway.
template <int MB, int NB, bool NORM>
struct SkinnyOperands {
    bf16x8 w[NB];
    bf16x8 x[NORM ? 1 : MB];
    f32x4 xf[NORM ? MB : 1][2];
    f32x4 g[2];
};

// An RMSNorm handed from the product before it to the product after it, for at most 16 rows:
//   RMSNorm(x; g) W^T = inv * (bf16(x * g) W^T),  inv = 1 / sqrt(sum(x^2) / width + eps) per row.
// The product that adds to the residual stream x (epilogue 1) also leaves xg = bf16(x * g) and,
// for every block of 16 columns, the sum of x^2 over the block (emit_*); the product that follows
// reads xg as its input and scales its sums by inv, which it gets by adding up those partial
// sums in a fixed order (scale_*). No norm kernel runs in between.
// With more than 16 rows K is (often) cut into slices and a second kernel adds them up: it sees whole
// rows and does the whole norm (emit_partial null, emit_eps its eps; emit_xg is then the normed rows).
struct NormHandoff {
    const float* emit_g;         // weight of the norm that follows, [N]; null: nothing is left behind
    bf16* emit_xg;               // [M, N]
    float* emit_partial;         // [ceil(N / 16), MP], MP = M rounded up to a power of two; rows from M on hold zeros
    const float* scale_partial;  // [scale_parts, MP] of the product before; null: no scaling
    int scale_parts;
    float scale_eps;             // the width of the normed rows is this product's K
    float emit_eps;
};

template <int MB, int NB, int WAVES, int EPI, bool PACKED, bool NORM>
__global__ void __launch_bounds__(WAVES * 64)
gemm_skinny_kernel(const void* __restrict__ Xv, const bf16* __restrict__ W, void* __restrict__ Cv, int M,
                   int N, int K, int ldc, const float* __restrict__ norm_w, float eps, NormHandoff hand) {
    constexpr int U = NORM ? 2 : ((NB + MB <= 4) ? 4 : 2);
    const bf16* X = (const bf16*)Xv;
    const float* XF = (const float*)Xv;
    extern __shared__ float red[];   // [WAVES / 2][NB * MB * 4][64]
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int r16 = lane & 15;
    const int g4 = lane >> 4;
    const int n0 = blockIdx.x * (NB * 16);
    const int nsteps = K / 32;                    // k-steps of the product

    f32x4 acc[NB][MB];
#pragma unroll
    for (int a = 0; a < NB; ++a)
#pragma unroll
        for (int b = 0; b < MB; ++b) acc[a][b] = f32x4{0.f, 0.f, 0.f, 0.f};

    // row-major weights: lane (r16, g4) reads 16 bytes of row n at k = 32 s + 8 g4.
    // packed weights: the 1 KB operand of (block of 16 rows, k-step) is contiguous, lane-major.
    const bf16* wrow[NB];
    // elements between this lane's chunks of two k-steps: packed weights are [K / 32][N / 16][64][8]
    const size_t WSTEP = PACKED ? (size_t)(N / 16) * 512 : 32;
#pragma unroll
    for (int a = 0; a < NB; ++a) {
        if (PACKED) {
            int nb = n0 / 16 + a;
            if (nb * 16 >= N) nb = (N - 1) / 16;
            wrow[a] = W + ((size_t)nb * 64 + lane) * 8;
        } else {
            int n = n0 + a * 16 + r16;
            if (n >= N) n = N - 1;            // rows past the end repeat the last one; never stored
            wrow[a] = W + (size_t)n * K + g4 * 8;
        }
    }
    const bf16* xrow[MB];
    const float* xfrow[MB];
#pragma unroll
    for (int b = 0; b < MB; ++b) {
        int m = b * 16 + r16;
        if (m >= M) m = M - 1;
        xrow[b] = X + (size_t)m * K + g4 * 8;
        xfrow[b] = XF + (size_t)m * K + g4 * 8;
    }
    float sumsq[MB];
#pragma unroll
    for (int b = 0; b < MB; ++b) sumsq[b] = 0.f;
    // What wave 0 adds its sums to, and the norm weights it needs to leave a norm behind, are asked
    // for now: by the epilogue they have long arrived.
    float c_before[NB][4], g_ahead[NB][4];
    if (EPI == EPI_ADD && MB == 1 && wave == 0) {
#pragma unroll
        for (int a = 0; a < NB; ++a)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int n = n0 + a * 16 + g4 * 4 + i;
                const bool in = r16 < M && n < N;
                c_before[a][i] = in ? ((const float*)Cv)[(size_t)r16 * ldc + n] : 0.f;
                g_ahead[a][i] = in && hand.emit_g ? hand.emit_g[n] : 0.f;
            }
    }
    const int mine = wave < nsteps ? (nsteps - wave + WAVES - 1) / WAVES : 0;   // this wave's steps
    const int groups = mine / U;
    SkinnyOperands<MB, NB, NORM> cur[U], nxt[U];

#define SKINNY_LOAD(dst, group)                                                  \
    _Pragma("unroll") for (int u = 0; u < U; ++u) {                              \
        const int st = wave + ((group) * U + u) * WAVES;                         \
        const int k = st * 32;                                                   \
        _Pragma("unroll") for (int a = 0; a < NB; ++a)                           \
            dst[u].w[a] = *(const bf16x8*)(wrow[a] + (size_t)st * WSTEP);        \
        if (NORM) {                                                              \
            dst[u].g[0] = *(const f32x4*)(norm_w + k + g4 * 8);                  \
            dst[u].g[1] = *(const f32x4*)(norm_w + k + g4 * 8 + 4);              \
            _Pragma("unroll") for (int b = 0; b < MB; ++b) {                     \
                dst[u].xf[b][0] = *(const f32x4*)(xfrow[b] + k);                 \
                dst[u].xf[b][1] = *(const f32x4*)(xfrow[b] + k + 4);             \
            }                                                                    \
        } else {                                                                 \
            _Pragma("unroll") for (int b = 0; b < MB; ++b)                       \
                dst[u].x[b] = *(const bf16x8*)(xrow[b] + k);                     \
        }                                                                        \
    }
#define SKINNY_MULTIPLY(src)                                                     \
    _Pragma("unroll") for (int u = 0; u < U; ++u)                                \
        _Pragma("unroll") for (int b = 0; b < MB; ++b) {                         \
            bf16x8 xop;                                                          \
            if (NORM) {                                                          \
                xop = normed_operand(src[u].xf[b], src[u].g, sumsq[b]);          \
            } else {                                                             \
                xop = src[u].x[b];                                               \
            }                                                                    \
            _Pragma("unroll") for (int a = 0; a < NB; ++a)                       \
                acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(src[u].w[a], xop, acc[a][b], 0, 0, 0); \
        }

    if (groups > 0) { SKINNY_LOAD(cur, 0) }
    // The row's sums of squares from the product before, [parts][MP], MP = the rows rounded up to a
    // power of two: thread t takes row t % MP of the parts t / MP, t / MP + threads / MP, ...; the
    // first HP of them are asked for here, behind the first weights, and land while the weights
    // stream; the sum is formed in the epilogue.
    constexpr int HP = 8;
    float hp[HP];
    const int MP = M <= 1 ? 1 : (M <= 2 ? 2 : (M <= 4 ? 4 : (M <= 8 ? 8 : 16)));
    const int hp_first = (int)threadIdx.x / MP, hp_step = WAVES * 64 / MP;
    if (MB == 1 && hand.scale_partial) {
#pragma unroll
        for (int j = 0; j < HP; ++j) {
            const int p = hp_first + j * hp_step;
            hp[j] = hand.scale_partial[(size_t)(p < hand.scale_parts ? p : hand.scale_parts - 1) * MP + (lane & (MP - 1))];
        }
    }
    for (int g = 0; g < groups; g += 2) {
        if (g + 1 < groups) { SKINNY_LOAD(nxt, g + 1) }
        SKINNY_MULTIPLY(cur)
        if (g + 1 < groups) {
            if (g + 2 < groups) { SKINNY_LOAD(cur, g + 2) }
            SKINNY_MULTIPLY(nxt)
        }
    }
    for (int i = groups * U; i < mine; ++i) {       // what is left over of this wave's steps
        const int st = wave + i * WAVES;
        const int k = st * 32;
        bf16x8 wv[NB], xv[MB];
#pragma unroll
        for (int a = 0; a < NB; ++a) wv[a] = *(const bf16x8*)(wrow[a] + (size_t)st * WSTEP);
#pragma unroll
        for (int b = 0; b < MB; ++b) {
            if (NORM) {
                f32x4 xf[2] = {*(const f32x4*)(xfrow[b] + k), *(const f32x4*)(xfrow[b] + k + 4)};
                f32x4 gg[2] = {*(const f32x4*)(norm_w + k + g4 * 8), *(const f32x4*)(norm_w + k + g4 * 8 + 4)};
                xv[b] = normed_operand(xf, gg, sumsq[b]);
            } else {
                xv[b] = *(const bf16x8*)(xrow[b] + k);
            }
        }
#pragma unroll
        for (int a = 0; a < NB; ++a)
#pragma unroll
            for (int b = 0; b < MB; ++b)
                acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wv[a], xv[b], acc[a][b], 0, 0, 0);
    }
#undef SKINNY_LOAD
#undef SKINNY_MULTIPLY

    // a fixed tree over the waves: the upper half adds into the lower half, until wave 0 holds all
    constexpr int REGS = NB * MB * 4;
    float inv_rms[MB];
    if (NORM) {
        // a row's squares: over the four lane groups of this wave, then over the waves in order
#pragma unroll
        for (int b = 0; b < MB; ++b) {
            sumsq[b] += __shfl_xor(sumsq[b], 16, 64);
            sumsq[b] += __shfl_xor(sumsq[b], 32, 64);
            if (lane < 16) red[(wave * MB + b) * 16 + lane] = sumsq[b];
        }
        __syncthreads();
#pragma unroll
        for (int b = 0; b < MB; ++b) {
            float total = 0.f;
            for (int w = 0; w < WAVES; ++w) total += red[(w * MB + b) * 16 + r16];
            inv_rms[b] = 1.0f / sqrtf(total / (float)K + eps);
        }
        __syncthreads();
    }
    float* handed_of_wave = red + (size_t)(WAVES / 2) * REGS * 64;   // [WAVES][16], behind the tree's space
    if (MB == 1 && hand.scale_partial) {
        float handed = 0.f;
#pragma unroll
        for (int j = 0; j < HP; ++j)     // past the end the last part was read once more: left out here
            handed += hp_first + j * hp_step < hand.scale_parts ? hp[j] : 0.f;
        // (what lies beyond the first HP parts of a thread, for long rows: asked for HP at a time too)
        for (int base = hp_first + HP * hp_step; base < hand.scale_parts; base += HP * hp_step) {
            float more[HP];
#pragma unroll
            for (int j = 0; j < HP; ++j) {
                const int p = base + j * hp_step;
                more[j] = hand.scale_partial[(size_t)(p < hand.scale_parts ? p : hand.scale_parts - 1) * MP + (lane & (MP - 1))];
            }
#pragma unroll
            for (int j = 0; j < HP; ++j) handed += base + j * hp_step < hand.scale_parts ? more[j] : 0.f;
        }
        for (int d = 32; d >= MP; d >>= 1) handed += __shfl_xor(handed, d, 64);   // lanes of the same row
        if (lane < MP) handed_of_wave[wave * 16 + lane] = handed;    // read by wave 0 after the tree's barriers
    }
#pragma unroll
    for (int half = WAVES / 2; half >= 1; half >>= 1) {
        if (wave >= half && wave < 2 * half) {
            float* dst = red + (size_t)(wave - half) * REGS * 64;
#pragma unroll
            for (int a = 0; a < NB; ++a)
#pragma unroll
                for (int b = 0; b < MB; ++b)
#pragma unroll
                    for (int i = 0; i < 4; ++i) dst[((a * MB + b) * 4 + i) * 64 + lane] = acc[a][b][i];
        }
        __syncthreads();
        if (wave < half) {
            const float* src = red + (size_t)wave * REGS * 64;
#pragma unroll
            for (int a = 0; a < NB; ++a)
#pragma unroll
                for (int b = 0; b < MB; ++b)
#pragma unroll
                    for (int i = 0; i < 4; ++i) acc[a][b][i] += src[((a * MB + b) * 4 + i) * 64 + lane];
        }
        __syncthreads();
    }
    if (wave != 0) return;
    if (NORM) {
#pragma unroll
        for (int a = 0; a < NB; ++a)
#pragma unroll
            for (int b = 0; b < MB; ++b)
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[a][b][i] *= inv_rms[b];
    }
    if (MB == 1 && hand.scale_partial) {
        float handed = 0.f;
        for (int w = 0; w < WAVES; ++w) handed += handed_of_wave[w * 16 + (r16 & (MP - 1))];
        const float inv = 1.0f / sqrtf(handed / (float)K + hand.scale_eps);
#pragma unroll
        for (int a = 0; a < NB; ++a)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[a][0][i] *= inv;
    }

    // lane: m = b * 16 + r16, n = n0 + a * 16 + g4 * 4 + i
    if (EPI == EPI_SWIGLU) {
        bf16* C = (bf16*)Cv;
        const int out_n0 = n0 / 2;
#pragma unroll
        for (int a = 0; a + 1 < NB; a += 2)
#pragma unroll
            for (int b = 0; b < MB; ++b) {
                const int m = b * 16 + r16;
                if (m >= M) continue;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int n = out_n0 + (a / 2) * 16 + g4 * 4 + i;
                    if (n < N / 2)
                        C[(size_t)m * ldc + n] = hb_from_float<bf16>(silu_mul(acc[a][b][i], acc[a + 1][b][i]));
                }
            }
    } else {
        float* C = (float*)Cv;
        const bool emit = EPI == EPI_ADD && MB == 1 && hand.emit_g;
#pragma unroll
        for (int a = 0; a < NB; ++a) {
            float squares = 0.f;      // of the new x over this lane's 4 of the block's 16 columns
#pragma unroll
            for (int b = 0; b < MB; ++b) {
                const int m = b * 16 + r16;
                if (m >= M) continue;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int n = n0 + a * 16 + g4 * 4 + i;
                    if (n < N) {
                        const size_t idx = (size_t)m * ldc + n;
                        float x = acc[a][b][i];
                        if (EPI == EPI_ADD) x += MB == 1 ? c_before[a][i] : C[idx];
                        C[idx] = x;
                        if (emit) {
                            squares = fmaf(x, x, squares);
                            hand.emit_xg[(size_t)m * N + n] = hb_from_float<bf16>(x * g_ahead[a][i]);
                        }
                    }
                }
            }
            if (emit) {               // the same for the whole wave
                squares += __shfl_xor(squares, 16, 64);
                squares += __shfl_xor(squares, 32, 64);
                const int block = n0 / 16 + a;
                if (g4 == 0 && r16 < MP && block * 16 < N) hand.emit_partial[(size_t)block * MP + r16] = squares;
            }
        }
    }
}

// C[m, n] (+)= sum over the slices, in their order, of partial[slice][m][n].
__global__ void gemm_slices_kernel(const float* __restrict__ partial, float* __restrict__ C, int M, int N,
                                   int ldc, int slices, int add) {
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (size_t)M * N) return;
    const int m = (int)(idx / N), n = (int)(idx % N);
    float sum = add ? C[(size_t)m * ldc + n] : 0.f;
    for (int s = 0; s < slices; ++s) sum += partial[(size_t)s * M * N + idx];
    C[(size_t)m * ldc + n] = sum;
}

// The same for a product that adds to the residual stream and is followed by an RMSNorm: a block a
// row adds the slices to x, stores x and writes y = bf16(x / rms(x) * g) as well (or, for at most 16
// rows, what NormHandoff describes: the next product expects that). A thread has at
// most CHUNKS chunks of four columns (N in steps of 4, at most 8192 = 4 THREADS CHUNKS) and asks for
// its part of up to FLY slices at once: with at most 64 rows there are few blocks, and what counts is
// that each has all its loads in flight together (1024 threads, eight slices); with many rows
// there are blocks enough, of 256 threads.
template <int THREADS, int CHUNKS, int FLY>
__global__ void __launch_bounds__(THREADS)
gemm_slices_norm_kernel(const float* __restrict__ partial, float* __restrict__ C, int M, int N, int ldc, int slices,
                        const float* __restrict__ g, float eps, bf16* __restrict__ y, float* __restrict__ squares) {
    __shared__ float red[16];
    const int m = blockIdx.x;
    f32x4* row = (f32x4*)(C + (size_t)m * ldc);
    const f32x4* g4 = (const f32x4*)g;
    const int nv = N / 4;
    f32x4 v[CHUNKS], gv[CHUNKS];
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int i = threadIdx.x + THREADS * c;
        const int at = i < nv ? i : nv - 1;              // past the end: the last chunk again, never stored
        v[c] = row[at];
        gv[c] = g4[at];
    }
    for (int s0 = 0; s0 < slices; s0 += FLY) {
        f32x4 p[CHUNKS][FLY];
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c) {
            const int i = threadIdx.x + THREADS * c;
            const int at = i < nv ? i : nv - 1;
#pragma unroll
            for (int j = 0; j < FLY; ++j) {
                const int sl = s0 + j < slices ? s0 + j : slices - 1;
                p[c][j] = ((const f32x4*)(partial + ((size_t)sl * M + m) * N))[at];
            }
        }
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c)
#pragma unroll
            for (int j = 0; j < FLY; ++j)
                if (s0 + j < slices) v[c] += p[c][j];     // in the order of the slices
    }
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int i = threadIdx.x + THREADS * c;
        if (i < nv) {
            row[i] = v[c];
            ss += v[c][0] * v[c][0] + v[c][1] * v[c][1] + v[c][2] * v[c][2] + v[c][3] * v[c][3];
        }
    }
    bf16* out = y + (size_t)m * N;
    if (squares) {
        // half the norm, as the few-row kernel leaves it (at most 16 rows): y = bf16(x * g) and the
        // sums of x^2 by blocks of 16 columns, four threads a block
        const int MP = M <= 1 ? 1 : (M <= 2 ? 2 : (M <= 4 ? 4 : (M <= 8 ? 8 : 16)));
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c) {
            const int i = threadIdx.x + THREADS * c;
            float sq = i < nv ? v[c][0] * v[c][0] + v[c][1] * v[c][1] + v[c][2] * v[c][2] + v[c][3] * v[c][3] : 0.f;
            sq += __shfl_xor(sq, 1, 64);
            sq += __shfl_xor(sq, 2, 64);
            if (i < nv) {
                if ((i & 3) == 0) squares[(size_t)(i / 4) * MP + m] = sq;
                bf16x4 o;
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = (__bf16)(v[c][e] * gv[c][e]);
                *(bf16x4*)((__bf16*)out + 4 * i) = o;
            }
        }
        if (m == 0)            // rows from M on hold zeros
            for (int i = threadIdx.x; i < (N + 15) / 16 * (MP - M); i += THREADS)
                squares[(size_t)(i / (MP - M)) * MP + M + i % (MP - M)] = 0.f;
        return;
    }
    ss = hb_block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)N + eps);
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int i = threadIdx.x + THREADS * c;
        if (i < nv) {
            bf16x4 o;
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = (__bf16)(v[c][e] * inv * gv[c][e]);
            *(bf16x4*)((__bf16*)out + 4 * i) = o;
        }
    }
}

// The same for the SwiGLU epilogue: column j of the output pairs the sums of the gate row
// 32 (j / 16) + j % 16 and of the up row 16 further on; C bf16 [M, N / 2].
__global__ void gemm_slices_swiglu_kernel(const float* __restrict__ partial, bf16* __restrict__ C, int M, int N,
                                          int ldc, int slices) {
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int half = N / 2;
    if (idx >= (size_t)M * half) return;
    const int m = (int)(idx / half), j = (int)(idx % half);
    const size_t at = (size_t)m * N + 32 * (j / 16) + j % 16;
    float gate = 0.f, up = 0.f;
    for (int s = 0; s < slices; ++s) {
        gate += partial[(size_t)s * M * N + at];
        up += partial[(size_t)s * M * N + at + 16];
    }
    C[(size_t)m * ldc + j] = hb_from_float<bf16>(silu_mul(gate, up));
}

template <int MB, int NB, int WAVES>
static void launch_skinny(const void* X, const void* W, void* C, int M, int N, int K, int ldc, int epi,
                          int packed, const float* norm_w, float eps, hipStream_t stream, const NormHandoff& hand) {
    const dim3 blocks((N + NB * 16 - 1) / (NB * 16));
    size_t lds = (size_t)(WAVES / 2) * NB * MB * 4 * 64 * sizeof(float);
    if (lds < (size_t)WAVES * MB * 16 * sizeof(float)) lds = (size_t)WAVES * MB * 16 * sizeof(float);
    lds += (size_t)WAVES * 16 * sizeof(float);      // a handed-on norm's sums, one row of 16 a wave
    const bf16* w = (const bf16*)W;
#define SKINNY_GO(EPIV, PK, NM)                                                                        \
    gemm_skinny_kernel<MB, NB, WAVES, EPIV, PK, NM><<<blocks, WAVES * 64, lds, stream>>>(X, w, C, M, N, K, \
                                                                                          ldc, norm_w, eps, hand)
    if (norm_w) {       // the normed input never meets the add epilogue; built for one block of rows
        if constexpr (MB == 1 && WAVES == 4) {
            if (packed) {
                if (epi == EPI_STORE) SKINNY_GO(EPI_STORE, true, true);
                else SKINNY_GO(EPI_SWIGLU, true, true);
            } else {
                if (epi == EPI_STORE) SKINNY_GO(EPI_STORE, false, true);
                else SKINNY_GO(EPI_SWIGLU, false, true);
            }
        }
    } else if (packed) {
        if (epi == EPI_STORE) SKINNY_GO(EPI_STORE, true, false);
        else if (epi == EPI_ADD) SKINNY_GO(EPI_ADD, true, false);
        else SKINNY_GO(EPI_SWIGLU, true, false);
    } else {
        if (epi == EPI_STORE) SKINNY_GO(EPI_STORE, false, false);
        else if (epi == EPI_ADD) SKINNY_GO(EPI_ADD, false, false);
        else SKINNY_GO(EPI_SWIGLU, false, false);
    }
#undef SKINNY_GO
}

// At most 16 rows. Few weight rows: one block of 16 rows a workgroup and eight waves splitting K,
// so that the 256 CUs all have work. Many rows: four blocks a workgroup.
static void pick_skinny(const void* X, const void* W, void* C, int M, int N, int K, int ldc, int epi,
                        int packed, const float* norm_w, float eps, hipStream_t stream, const NormHandoff& hand) {
    if (epi == EPI_SWIGLU || N >= 16384) {
        launch_skinny<1, 4, 4>(X, W, C, M, N, K, ldc, epi, packed, norm_w, eps, stream, hand);
    } else {
        launch_skinny<1, 1, 8>(X, W, C, M, N, K, ldc, epi, packed, norm_w, eps, stream, hand);
    }
}

// ------------------------------------------------------------------- tiled
// The product for many rows (prompts). Tiles go from global memory straight into LDS
// (hb_load_to_lds) through rings of stages that are loaded ahead of the MFMAs; what has landed
// is waited for by count (hb_wait_vmcnt) before a bare barrier (hb_workgroup_barrier).
// 32x32x16 MFMA (of the two bf16 shapes the one with the higher rate), weight rows first: an
// operand is 32 rows x 16 k, lane l = row l % 32, k 8 (l / 32) .. + 8; a lane ends with 16 sums
// of one m: n = 8 q + 4 (l / 32) + j for register 4 q + j.
// Weights lie in LDS as in memory when packed: 1 KB blocks of 16 rows x 32 k, chunk
// 16 (k / 8 % 4) + row % 16. For the k-half h of a k-step of 32 an operand is then: block
// (l % 32) / 16 of a pair of blocks, chunk 16 (2 h + l / 32) + l % 16: 16 lanes read 256
// contiguous bytes, free of bank conflicts.
// Workgroup: WNW x WMW waves, each TNB x TMB blocks of 16: BN = 16 TNB WNW, BM = 16 TMB WMW.
// Workgroups go round the 8 XCDs, each with an L2 of its own: an XCD takes a run of tiles, and
// within it bands of 8 tiles in m are walked n first, so that the workgroups that are resident
// together share both their weight and their activation panels in that L2.
__device__ __forceinline__ bool tile_of_workgroup(int m_tiles, int n_tiles, int& m_tile, int& n_tile) {
    const int total = m_tiles * n_tiles;
    const int chunk = (total + 7) / 8;
    const int id = (blockIdx.x % 8) * chunk + blockIdx.x / 8;
    if (id >= total) return false;
    constexpr int BAND = 8;
    const int band = id / (BAND * n_tiles), in_band = id % (BAND * n_tiles);
    const int band_rows = m_tiles - band * BAND < BAND ? m_tiles - band * BAND : BAND;
    n_tile = in_band / band_rows;
    m_tile = band * BAND + in_band % band_rows;
    return true;
}

// A wave's sums to memory. m_base, n_base: first row and column of the wave's tile.
template <int EPI, int TN32, int TM32>
__device__ __forceinline__ void store_wave_tile(const f32x16 (&acc)[TN32][TM32], void* Cv, int M, int N, int ldc,
                                                int m_base, int n_base, int c32, int g2) {
#pragma unroll
    for (int b = 0; b < TM32; ++b) {
        const int m = m_base + 32 * b + c32;
        if (m >= M) continue;
        if (EPI == EPI_SWIGLU) {
            bf16* C = (bf16*)Cv;
#pragma unroll
            for (int a = 0; a < TN32; ++a)
#pragma unroll
                for (int q = 0; q < 2; ++q) {
                    // rows 0..15 of a piece are gate rows, 16..31 the up rows of the same outputs
                    const int n = (n_base + 32 * a) / 2 + 8 * q + 4 * g2;
                    if (n + 3 < N / 2 && (ldc & 3) == 0) {
                        bf16x4 v;
#pragma unroll
                        for (int j = 0; j < 4; ++j)
                            v[j] = (__bf16)silu_mul(acc[a][b][4 * q + j], acc[a][b][4 * q + 8 + j]);
                        *(bf16x4*)((__bf16*)C + (size_t)m * ldc + n) = v;
                    } else {
#pragma unroll
                        for (int j = 0; j < 4; ++j)
                            if (n + j < N / 2)
                                C[(size_t)m * ldc + n + j] = hb_from_float<bf16>(
                                    silu_mul(acc[a][b][4 * q + j], acc[a][b][4 * q + 8 + j]));
                    }
                }
        } else {
            float* C = (float*)Cv;
#pragma unroll
            for (int a = 0; a < TN32; ++a)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int n = n_base + 32 * a + 8 * q + 4 * g2;
                    float* dst = C + (size_t)m * ldc + n;
                    if (n + 3 < N && (ldc & 3) == 0) {
                        f32x4 v = {acc[a][b][4 * q], acc[a][b][4 * q + 1], acc[a][b][4 * q + 2],
                                   acc[a][b][4 * q + 3]};
                        if (EPI == EPI_ADD) v += *(const f32x4*)dst;
                        *(f32x4*)dst = v;
                    } else {
#pragma unroll
                        for (int j = 0; j < 4; ++j)
                            if (n + j < N) {
                                if (EPI == EPI_ADD)
                                    dst[j] += acc[a][b][4 * q + j];
                                else
                                    dst[j] = acc[a][b][4 * q + j];
                            }
                    }
                }
        }
    }
}

// The same through LDS, for float32 outputs of the large tiles: a lane's sums are runs of four
// columns of 32 different rows, so a store instruction of the direct way touches 32 lines in
// pieces of 32 bytes, and reading C back for the add does the same (a round of 256 x 256 tiles
// spent 45 us beside its products with the store and 68 us with the add, against 19 us with the
// bfloat16 SwiGLU output). Here a wave first lays PB x 32 rows of its tile into LDS of its own
// (`stage`, rows of TN32 x 32 floats, the 16-byte chunk c of row r at chunk c ^ (r mod chunks)),
// then reads them back along the rows: an instruction then moves whole rows, 512 contiguous
// bytes for a tile 128 wide. Needs ldc and N in steps of 4 and C aligned to 16 bytes.
template <int EPI, int TN32, int TM32, int PB>
__device__ __forceinline__ void store_wave_tile_lds(const f32x16 (&acc)[TN32][TM32], float* C, int M, int N, int ldc,
                                                    int m_base, int n_base, int lane, float* stage) {
    static_assert(TM32 % PB == 0, "the passes divide the wave's tile");
    constexpr int CH = TN32 * 8;            // 16-byte chunks of a row
    constexpr int RPI = 64 / CH;            // rows an instruction moves
    constexpr int ITER = PB * 32 / RPI;
    constexpr int GROUP = ITER < 8 ? ITER : 8;
    const int c32 = lane & 31, g2 = lane >> 5;
    const int rrow = lane / CH, rchunk = lane % CH;
#pragma unroll
    for (int b0 = 0; b0 < TM32; b0 += PB) {
#pragma unroll
        for (int bb = 0; bb < PB; ++bb)
#pragma unroll
            for (int a = 0; a < TN32; ++a)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int row = 32 * bb + c32, chunk = 8 * a + 2 * q + g2;
                    const f32x4 v = {acc[a][b0 + bb][4 * q], acc[a][b0 + bb][4 * q + 1], acc[a][b0 + bb][4 * q + 2],
                                     acc[a][b0 + bb][4 * q + 3]};
                    *(f32x4*)(stage + row * (CH * 4) + ((chunk ^ (row & (CH - 1))) * 4)) = v;
                }
#pragma unroll
        for (int i0 = 0; i0 < ITER; i0 += GROUP) {
            f32x4 before[GROUP];
            if (EPI == EPI_ADD) {
#pragma unroll
                for (int u = 0; u < GROUP; ++u) {
                    const int row = (i0 + u) * RPI + rrow;
                    const int m = m_base + 32 * b0 + row, n = n_base + 4 * rchunk;
                    before[u] = (m < M && n < N) ? *(const f32x4*)(C + (size_t)m * ldc + n) : f32x4{0.f, 0.f, 0.f, 0.f};
                }
            }
#pragma unroll
            for (int u = 0; u < GROUP; ++u) {
                const int row = (i0 + u) * RPI + rrow;
                const int m = m_base + 32 * b0 + row, n = n_base + 4 * rchunk;
                f32x4 v = *(const f32x4*)(stage + row * (CH * 4) + ((rchunk ^ (row & (CH - 1))) * 4));
                if (EPI == EPI_ADD) v += before[u];
                if (m < M && n < N) *(f32x4*)(C + (size_t)m * ldc + n) = v;
            }
        }
    }
}

// The SwiGLU outputs of the large tiles through LDS as well. A lane holds runs of four outputs of
// 32 different rows, 8 bytes each: a store instruction of the direct way touches 32 lines in pieces
// of 16 bytes (a round of 256 x 256 tiles spent 15 us beside its products that way, for a quarter
// of the bytes that the float32 store moves in 8). Here a wave lays its whole tile's outputs into
// LDS of its own (rows of TN32 x 16 bfloat16, the 16-byte chunk c of row r at chunk c ^ (r mod
// chunks), or (c + r) mod chunks where the chunks are no power of two), then reads them back
// along the rows: an instruction stores whole rows, 128 contiguous bytes for a tile 128 wide.
// n_base: the wave's first column among the interleaved gate/up columns. Needs ldc in steps of
// 8 and C aligned to 16 bytes.
template <int TN32, int TM32>
__device__ __forceinline__ void store_wave_tile_swiglu_lds(const f32x16 (&acc)[TN32][TM32], bf16* C, int M, int N,
                                                           int ldc, int m_base, int n_base, int lane, bf16* stage) {
    constexpr int CH = 2 * TN32;            // 16-byte chunks of a row: 16 outputs a piece of 32 columns
    constexpr int RPI = 64 / CH;            // rows an instruction moves
    constexpr int ROWS = 32 * TM32;
    constexpr bool POW2 = (CH & (CH - 1)) == 0;
    auto place = [&](int row, int chunk) { return POW2 ? (chunk ^ (row & (CH - 1))) : (chunk + row) % CH; };
    const int c32 = lane & 31, g2 = lane >> 5;
#pragma unroll
    for (int b = 0; b < TM32; ++b)
#pragma unroll
        for (int a = 0; a < TN32; ++a)
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                // rows 0..15 of a piece are gate rows, 16..31 the up rows of the same outputs
                const int row = 32 * b + c32;
                bf16x4 v;
#pragma unroll
                for (int j = 0; j < 4; ++j) v[j] = (__bf16)silu_mul(acc[a][b][4 * q + j], acc[a][b][4 * q + 8 + j]);
                *(bf16x4*)((__bf16*)stage + row * (CH * 8) + place(row, 2 * a + q) * 8 + 4 * g2) = v;
            }
    const int rrow = lane / CH, rchunk = lane % CH;
    if (lane >= RPI * CH) return;
#pragma unroll
    for (int i = 0; i < (ROWS + RPI - 1) / RPI; ++i) {
        const int row = i * RPI + rrow;
        if (row >= ROWS) break;
        const int m = m_base + row, n = n_base / 2 + 8 * rchunk;
        const bf16x8 v = *(const bf16x8*)((const __bf16*)stage + row * (CH * 8) + place(row, rchunk) * 8);
        if (m >= M) continue;
        if (n + 7 < N / 2) {
            *(bf16x8*)((__bf16*)C + (size_t)m * ldc + n) = v;
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j)
                if (n + j < N / 2) ((__bf16*)C)[(size_t)m * ldc + n + j] = v[j];
        }
    }
}

// The q/k/v projection of prompts with what follows it, for heads of 128 (a wave's tile is 128
// columns wide: one head): per-head RMSNorm (if weights are given), rotation over the whole head
// (if tables are given), queries to q_out [M, nq 128] and keys and values into the pages (values
// transposed), all bfloat16. The float32 sums never go to memory.
struct QkvEpilogue {
    bf16* q_out;
    bf16* k_cache;               // [pages, nkv, 64, 128]
    bf16* v_cache;               // [pages, nkv, 128, 64]
    const int* positions;        // of every row
    const int* seq_of;           // row -> sequence of the step
    const int* slots;            // sequence -> slot
    const int* page_table;       // [slots, max_pages]
    int max_pages;
    const float* q_norm_w;
    const float* k_norm_w;
    const float* cos_t;          // [positions, 64]
    const float* sin_t;
    float eps;
    int nq, nkv;
};

// lane: row m = m_base + 32 b + c32; register 4 q + j of piece a: element 32 a + 8 q + 4 g2 + j of the head
template <int TN32, int TM32>
__device__ __forceinline__ void store_wave_tile_qkv(f32x16 (&acc)[TN32][TM32], const QkvEpilogue& e, int M, int N,
                                                    int m_base, int n_base, int c32, int g2) {
    static_assert(TN32 == 4, "a wave's tile must be one head of 128 wide");
    if (n_base >= N) return;
    const int head = n_base / 128;
    const bool is_q = head < e.nq, is_v = head >= e.nq + e.nkv;
    const float* norm_w = is_q ? e.q_norm_w : e.k_norm_w;
#pragma unroll
    for (int b = 0; b < TM32; ++b) {
        const int m = m_base + 32 * b + c32;
        const int mc = m < M ? m : M - 1;
        const int pos = e.positions[mc];
        if (!is_v) {
            if (norm_w) {
                float ss = 0.f;
#pragma unroll
                for (int a = 0; a < 4; ++a)
#pragma unroll
                    for (int i = 0; i < 16; ++i) ss = fmaf(acc[a][b][i], acc[a][b][i], ss);
                ss += __shfl_xor(ss, 32, 64);
                const float inv = 1.0f / sqrtf(ss / 128.0f + e.eps);
#pragma unroll
                for (int a = 0; a < 4; ++a)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const f32x4 w = *(const f32x4*)(norm_w + 32 * a + 8 * q + 4 * g2);
#pragma unroll
                        for (int j = 0; j < 4; ++j) acc[a][b][4 * q + j] = acc[a][b][4 * q + j] * inv * w[j];
                    }
            }
            if (e.cos_t) {
                // element d < 64 pairs with d + 64: pieces a and a + 2, the same register
#pragma unroll
                for (int a = 0; a < 2; ++a)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const size_t at = (size_t)pos * 64 + 32 * a + 8 * q + 4 * g2;
                        const f32x4 c = *(const f32x4*)(e.cos_t + at), s = *(const f32x4*)(e.sin_t + at);
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            const float x0 = acc[a][b][4 * q + j], x1 = acc[a + 2][b][4 * q + j];
                            acc[a][b][4 * q + j] = x0 * c[j] - x1 * s[j];
                            acc[a + 2][b][4 * q + j] = x0 * s[j] + x1 * c[j];
                        }
                    }
            }
        }
        if (m >= M) continue;
        if (is_q) {
            bf16* dst = e.q_out + ((size_t)m * e.nq + head) * 128;
#pragma unroll
            for (int a = 0; a < 4; ++a)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    bf16x4 v;
#pragma unroll
                    for (int j = 0; j < 4; ++j) v[j] = (__bf16)acc[a][b][4 * q + j];
                    *(bf16x4*)((__bf16*)dst + 32 * a + 8 * q + 4 * g2) = v;
                }
            continue;
        }
        const int page = e.page_table[(size_t)e.slots[e.seq_of[m]] * e.max_pages + pos / 64];
        const int in_page = pos % 64;
        if (!is_v) {
            bf16* dst = e.k_cache + (((size_t)page * e.nkv + (head - e.nq)) * 64 + in_page) * 128;
#pragma unroll
            for (int a = 0; a < 4; ++a)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    bf16x4 v;
#pragma unroll
                    for (int j = 0; j < 4; ++j) v[j] = (__bf16)acc[a][b][4 * q + j];
                    *(bf16x4*)((__bf16*)dst + 32 * a + 8 * q + 4 * g2) = v;
                }
        } else {
            // transposed pages: for one element the 32 lanes of a half wave write 32 neighbouring tokens
            bf16* dst = e.v_cache + ((size_t)page * e.nkv + (head - e.nq - e.nkv)) * 128 * 64 + in_page;
#pragma unroll
            for (int a = 0; a < 4; ++a)
#pragma unroll
                for (int i = 0; i < 16; ++i)
                    dst[(size_t)(32 * a + 8 * (i >> 2) + 4 * g2 + (i & 3)) * 64] = hb_from_float<bf16>(acc[a][b][i]);
        }
    }
}

// The second half of a handed-on norm (see NormHandoff) for the tiled product: at most 16 rows.
struct RowScale {
    const float* partial;        // [parts, MP]; null: no scaling
    int parts;
    float eps;
};

// K in steps of 64. A step's weights are two k-steps of 32 (blocks as above); its activations lie
// in LDS as rows of 128 bytes, so that a load fetches whole 128-byte lines (8 rows an
// instruction, 8 lanes a row) and not half lines twice; the 16-byte chunk c of row r sits at
// chunk c ^ ((r >> 1) & 7) of its row, so that the operand reads of 16 rows at one k fall into
// 16 different bank groups. The weights have a ring of WST stages, the activations one of XST.
// There is no branch in the main loop (the last step is peeled off), and what is no MFMA is
// dealt out between the MFMAs by hand: a wave has an MFMA in the pipe while it issues its reads
// and loads, also right after the barrier, where no other wave could fill in. Operands are in
// two sets of registers: the reads of a k-step go out during the MFMAs of the one before.
template <int EPI, bool PACKED, int TNB, int TMB, int WNW, int WMW, int WST, int XST>
__global__ void __launch_bounds__(64 * WNW * WMW)
gemm_tile_kernel(const bf16* __restrict__ X, const bf16* __restrict__ W, void* __restrict__ Cv, int M, int N,
                 int K, int ldc, int m_tiles, int n_tiles, float* __restrict__ partial, QkvEpilogue qkv,
                 RowScale scale) {
    constexpr int NW = WNW * WMW;
    constexpr int BN = 16 * TNB * WNW, BM = 16 * TMB * WMW;
    constexpr int WBLK = BN / 16;                       // weight blocks of a k-step of 32
    constexpr int WL = WBLK / NW;                       // of which a wave loads
    constexpr int XR = BM / 8 / NW;                     // loads of 8 activation rows of a wave per step
    constexpr int W_STAGE = 2 * WBLK * 512, X_STAGE = BM * 64;      // elements
    constexpr int NLW = 2 * WL, NLX = XR;               // a wave's loads per step
    static_assert(WBLK % NW == 0 && BM % (8 * NW) == 0, "the loads must divide over the waves");
    static_assert(TNB % 2 == 0 && TMB % 2 == 0, "a wave's tile is made of 32 x 32 pieces");
    static_assert((WST == 2 || WST == 3) && (XST == 2 || XST == 3),
                  "the wait before the barrier counts on the loads of at most one later step");
    constexpr bool X_FIRST = XST <= WST;                // in a step's loads: the operand with the shorter ring first
    constexpr int LATER = (WST == 3 ? NLW : 0) + (XST == 3 ? NLX : 0);   // loads that may be in flight at the barrier
    constexpr int TN32 = TNB / 2, TM32 = TMB / 2;
    extern __shared__ __attribute__((aligned(1024))) bf16 lds[];    // [WST][W_STAGE], then [XST][X_STAGE]
    bf16* const xlds = lds + WST * W_STAGE;

    int m_tile, n_tile;
    if (!tile_of_workgroup(m_tiles, n_tiles, m_tile, n_tile)) return;
    const int m0 = m_tile * BM, n0 = n_tile * BN;
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // uniform: LDS addresses stay scalar
    const int r16 = lane & 15, g4 = lane >> 4, c32 = lane & 31, g2 = lane >> 5;
    const int wn = wave / WMW, wm = wave % WMW;
    // gridDim.y > 1: K is cut into slices over workgroups (few tiles, long K); a workgroup leaves the
    // sums of its slice in `partial` [slice][M][N] and gemm_slices_kernel adds the slices in order
    const int all_steps = K / 64;
    const int per_slice = (all_steps + gridDim.y - 1) / gridDim.y;
    const int step0 = blockIdx.y * per_slice;
    const int nsteps = all_steps - step0 < per_slice ? all_steps - step0 : per_slice;    // >= 1: the host sees to it

    const size_t WSTEP = PACKED ? (size_t)(N / 16) * 512 : 32;      // elements between two k-steps of 32
    const bf16* wsrc[WL];
#pragma unroll
    for (int i = 0; i < WL; ++i) {
        const int blk = wave * WL + i;
        if (PACKED) {
            int nb = n0 / 16 + blk;
            if (nb * 16 >= N) nb = (N - 1) / 16;
            wsrc[i] = W + ((size_t)nb * 64 + lane) * 8 + (size_t)step0 * 2 * WSTEP;
        } else {
            int n = n0 + blk * 16 + r16;
            if (n >= N) n = N - 1;                      // rows past the end repeat the last one; never stored
            wsrc[i] = W + (size_t)n * K + g4 * 8 + (size_t)step0 * 2 * WSTEP;
        }
    }
    const bf16* xsrc[XR];
#pragma unroll
    for (int i = 0; i < XR; ++i) {
        const int r = (wave * XR + i) * 8 + (lane >> 3);
        int m = m0 + r;
        if (m >= M) m = M - 1;
        xsrc[i] = X + (size_t)m * K + (((lane & 7) ^ ((r >> 1) & 7)) * 8) + (size_t)step0 * 64;
    }
    // The idx-th load of a step: activations of step xstep into stage xstage, weights of step
    // wstep into stage wstage. The operand with the shorter ring comes first: it is the one
    // that is needed a step earlier.
    auto load_one = [&](int xstep, int xstage, int wstep, int wstage, int idx) {
        const bool is_x = X_FIRST ? idx < NLX : idx >= NLW;
        const int i = X_FIRST ? (is_x ? idx : idx - NLX) : (is_x ? idx - NLW : idx);
        if (is_x) {
            hb_load_to_lds(xsrc[i] + (size_t)xstep * 64, xlds + xstage * X_STAGE + (wave * XR + i) * 512);
        } else {
            const int ks = i / WL, w = i % WL;
            hb_load_to_lds(wsrc[w] + ((size_t)wstep * 2 + ks) * WSTEP,
                           lds + wstage * W_STAGE + ks * WBLK * 512 + (wave * WL + w) * 512);
        }
    };
    auto load_is_x = [&](int idx) { return X_FIRST ? idx < NLX : idx >= NLW; };

    f32x16 acc[TN32][TM32];
#pragma unroll
    for (int a = 0; a < TN32; ++a)
#pragma unroll
        for (int b = 0; b < TM32; ++b)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[a][b][i] = 0.f;

    constexpr int NM = 2 * TN32 * TM32;              // MFMAs of a k-step of 32
    constexpr int NR = 2 * (TN32 + TM32);            // operand reads of a k-step
    constexpr int SLOTS = NM > 6 ? NM - 4 : NM;      // the last MFMAs cover the latency of the last reads
    const int w_lane = (c32 >> 4) * 512 + (16 * g2 + (lane & 15)) * 8 + wn * TNB * 512;
    const int x_lane = (wm * TMB * 16 + c32) * 64;
    const int x_swizzle = (c32 >> 1) & 7;            // of this lane's rows: they are c32 + a multiple of 16
    bf16x8 wv[2][2][TN32], xv[2][2][TM32];           // [set][k-half][piece]
    auto mfma_one = [&](int set, int j) {
        const int h = j / (TN32 * TM32), a = j / TM32 % TN32, b = j % TM32;
        acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wv[set][h][a], xv[set][h][b], acc[a][b], 0, 0, 0);
    };
    auto read_one = [&](int set, int step, int ks, int idx) {
        const int h = idx / (TN32 + TM32), r = idx % (TN32 + TM32);
        if (r < TN32)
            wv[set][h][r] = *(const bf16x8*)(lds + (step % WST) * W_STAGE + ks * WBLK * 512 + w_lane + r * 1024 + h * 256);
        else
            xv[set][h][r - TN32] = *(const bf16x8*)(xlds + (step % XST) * X_STAGE + x_lane + (r - TN32) * 32 * 64 +
                                                    (((4 * ks + 2 * h + g2) ^ x_swizzle) * 8));
    };
    // between the MFMAs j and j + 1 of a k-step: nl loads and NR reads, dealt out evenly over the
    // first SLOTS MFMAs, the loads spread among the reads (a burst of loads from all waves at
    // once backs up the memory pipeline and holds the waves at their issue)
    auto between = [&](int j, int nl, auto&& load, auto&& read) {
        const int no = nl + NR;
        const int from = (j < SLOTS ? j : SLOTS) * no / SLOTS, to = (j + 1 < SLOTS ? j + 1 : SLOTS) * no / SLOTS;
#pragma unroll
        for (int o = from; o < to; ++o) {
            const int loads_before = o * nl / no, loads_after = (o + 1) * nl / no;
            if (loads_after > loads_before) load(loads_before);
            else read(o - loads_before);
        }
    };
    auto clamp = [&](int step) { return step < nsteps ? step : nsteps - 1; };   // past the end: the last step again

    // in flight before the loop: steps 0 and 1, and step 2 of what has a ring of three stages
#pragma unroll
    for (int i = 0; i < NLX + NLW; ++i) load_one(0, 0, 0, 0, i);
#pragma unroll
    for (int i = 0; i < NLX + NLW; ++i) load_one(clamp(1), 1, clamp(1), 1, i);
#pragma unroll
    for (int i = 0; i < NLX + NLW; ++i)
        if (load_is_x(i) ? XST == 3 : WST == 3) load_one(clamp(2), 2, clamp(2), 2, i);
    // A handed-on norm: every row's sum of squares is added up here, behind the first loads, by
    // all threads (thread t: row t % MP, parts t / MP, t / MP + threads / MP, ...), then over the
    // lanes of a row and, after the barrier, over the waves in their order.
    float* const row_sums = (float*)(xlds + XST * X_STAGE);       // [NW][16]
    const int MP = M <= 1 ? 1 : (M <= 2 ? 2 : (M <= 4 ? 4 : (M <= 8 ? 8 : 16)));
    if (scale.partial) {
        // (asked for HP at a time: one after another, as a plain loop over the parts does it, every
        // part costs a trip to the L2; with 16 rows and 256 parts that were eight trips, 8 us)
        constexpr int HP = 16;
        const int first = tid / MP, stride = 64 * NW / MP;
        float sum = 0.f;
        for (int base = first; base < scale.parts; base += HP * stride) {
            float hp[HP];
#pragma unroll
            for (int j = 0; j < HP; ++j) {
                const int p = base + j * stride;
                hp[j] = scale.partial[(size_t)(p < scale.parts ? p : scale.parts - 1) * MP + (lane & (MP - 1))];
            }
#pragma unroll
            for (int j = 0; j < HP; ++j) sum += base + j * stride < scale.parts ? hp[j] : 0.f;
        }
        for (int d = 32; d >= MP; d >>= 1) sum += __shfl_xor(sum, d, 64);
        if (lane < MP) row_sums[wave * 16 + lane] = sum;
    }
    hb_wait_vmcnt<NLX + NLW + LATER>();
    hb_workgroup_barrier();
    float inv_rms = 1.f;          // of row c32 (the scaled product has at most 16 rows, all in the first piece)
    if (scale.partial) {
        float sum = 0.f;
        for (int w = 0; w < NW; ++w) sum += row_sums[w * 16 + (c32 & (MP - 1))];
        inv_rms = 1.0f / sqrtf(sum / (float)K + scale.eps);
    }
#pragma unroll
    for (int i = 0; i < NR; ++i) read_one(0, 0, 0, i);

    for (int t = 0; t + 1 < nsteps; ++t) {
        // first k-step of step t; between its MFMAs the reads of the second one
#pragma unroll
        for (int j = 0; j < NM; ++j) {
            mfma_one(0, j);
            between(j, 0, [&](int) {}, [&](int i) { read_one(1, t, 1, i); });
            __builtin_amdgcn_sched_barrier(0);
        }
        // Step t + 1 has landed (of what this wave has in flight only the weights of the later
        // steps may be missing), after the barrier for every wave, and nobody reads step t any
        // more: between the MFMAs of its second k-step go the loads into its stages, the
        // activations of step t + XST and the weights of step t + WST, and the reads of step t + 1.
        hb_wait_vmcnt<LATER>();
        hb_workgroup_barrier();
        const int xstep = clamp(t + XST), wstep = clamp(t + WST);
#pragma unroll
        for (int j = 0; j < NM; ++j) {
            mfma_one(1, j);
            // (a clamped step goes where step t + XST or t + WST would: into the stage just freed)
            between(j, NLX + NLW, [&](int i) { load_one(xstep, t % XST, wstep, t % WST, i); },
                    [&](int i) { read_one(0, t + 1, 0, i); });
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    {
        const int t = nsteps - 1;
#pragma unroll
        for (int j = 0; j < NM; ++j) {
            mfma_one(0, j);
            between(j, 0, [&](int) {}, [&](int i) { read_one(1, t, 1, i); });
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int j = 0; j < NM; ++j) mfma_one(1, j);
    }
    hb_wait_vmcnt<0>();      // the loads past the end (repeats of the last step) have landed too
    if (scale.partial) {
#pragma unroll
        for (int a = 0; a < TN32; ++a)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[a][0][i] *= inv_rms;
    }
    if constexpr (EPI == EPI_QKV)
        store_wave_tile_qkv<TN32, TM32>(acc, qkv, M, N, m0 + wm * TMB * 16, n0 + wn * TNB * 16, c32, g2);
    else {
        // float32 outputs of the large tiles go through LDS (see store_wave_tile_lds): each wave has a
        // quarter of what the rings held, once every wave's loads have landed and its reads are done
        constexpr int REGION = (WST * W_STAGE + XST * X_STAGE) * (int)sizeof(bf16) / NW;       // bytes
        constexpr int PB_FIT = REGION / (32 * TN32 * 128);
        constexpr int PB = PB_FIT >= TM32 ? TM32 : (PB_FIT >= 2 && TM32 % 2 == 0 ? 2 : 1);
        constexpr bool VIA_LDS = (EPI == EPI_STORE || EPI == EPI_ADD) && BM >= 128 && PB_FIT >= 1;
        const bool sliced = gridDim.y > 1;
        float* const dst = sliced ? partial + (size_t)blockIdx.y * M * N : (float*)Cv;
        const int ld = sliced ? N : ldc;
        constexpr bool SWIGLU_VIA_LDS = EPI == EPI_SWIGLU && BM >= 128 && REGION >= 32 * TM32 * TN32 * 32;
        if (SWIGLU_VIA_LDS && !sliced && (ldc & 7) == 0 && ((size_t)Cv & 15) == 0) {
            hb_workgroup_barrier();
            store_wave_tile_swiglu_lds<TN32, TM32>(acc, (bf16*)Cv, M, N, ldc, m0 + wm * TMB * 16, n0 + wn * TNB * 16, lane,
                                                   (bf16*)((char*)lds + wave * REGION));
        } else if (VIA_LDS && (ld & 3) == 0 && (N & 3) == 0 && ((size_t)dst & 15) == 0) {
            hb_workgroup_barrier();
            float* const stage = (float*)((char*)lds + wave * REGION);
            if (sliced || EPI == EPI_STORE)
                store_wave_tile_lds<EPI_STORE, TN32, TM32, PB>(acc, dst, M, N, ld, m0 + wm * TMB * 16,
                                                               n0 + wn * TNB * 16, lane, stage);
            else
                store_wave_tile_lds<EPI_ADD, TN32, TM32, PB>(acc, dst, M, N, ld, m0 + wm * TMB * 16,
                                                             n0 + wn * TNB * 16, lane, stage);
        } else if (sliced) {
            store_wave_tile<EPI_STORE, TN32, TM32>(acc, dst, M, N, N, m0 + wm * TMB * 16, n0 + wn * TNB * 16, c32, g2);
        } else {
            store_wave_tile<EPI, TN32, TM32>(acc, Cv, M, N, ldc, m0 + wm * TMB * 16, n0 + wn * TNB * 16, c32, g2);
        }
    }
}

// K in steps of 32 only: one k-step a stage, everything in 1 KB blocks (the activations too: a
// block of 16 rows x 32 k is loaded as 16 half lines), a ring of STAGES stages loaded STAGES - 1
// steps ahead, the plain order read / multiply with the operands in two sets of registers.
template <int EPI, bool PACKED, int TNB, int TMB, int WNW, int WMW, int STAGES>
__global__ void __launch_bounds__(64 * WNW * WMW)
gemm_tile32_kernel(const bf16* __restrict__ X, const bf16* __restrict__ W, void* __restrict__ Cv, int M, int N,
                   int K, int ldc, int m_tiles, int n_tiles) {
    constexpr int NW = WNW * WMW;
    constexpr int BN = 16 * TNB * WNW, BM = 16 * TMB * WMW;
    constexpr int WBLK = BN / 16, XBLK = BM / 16, BLKS = WBLK + XBLK;   // 1 KB blocks of a stage
    constexpr int WL = WBLK / NW, XL = XBLK / NW;                      // loads of a wave per stage
    static_assert(WBLK % NW == 0 && XBLK % NW == 0, "blocks must divide over the waves");
    static_assert(TNB % 2 == 0 && TMB % 2 == 0, "a wave's tile is made of 32 x 32 pieces");
    constexpr int TN32 = TNB / 2, TM32 = TMB / 2;
    extern __shared__ __attribute__((aligned(1024))) bf16 lds[];        // [STAGES][BLKS][512]

    int m_tile, n_tile;
    if (!tile_of_workgroup(m_tiles, n_tiles, m_tile, n_tile)) return;
    const int m0 = m_tile * BM, n0 = n_tile * BN;
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r16 = lane & 15, g4 = lane >> 4, c32 = lane & 31, g2 = lane >> 5;
    const int wn = wave / WMW, wm = wave % WMW;
    const int nsteps = K / 32;

    const bf16* wsrc[WL];
    const bf16* xsrc[XL];
#pragma unroll
    for (int i = 0; i < WL; ++i) {
        const int blk = wave * WL + i;
        if (PACKED) {
            int nb = n0 / 16 + blk;
            if (nb * 16 >= N) nb = (N - 1) / 16;
            wsrc[i] = W + ((size_t)nb * 64 + lane) * 8;
        } else {
            int n = n0 + blk * 16 + r16;
            if (n >= N) n = N - 1;
            wsrc[i] = W + (size_t)n * K + g4 * 8;
        }
    }
#pragma unroll
    for (int i = 0; i < XL; ++i) {
        int m = m0 + (wave * XL + i) * 16 + r16;
        if (m >= M) m = M - 1;
        xsrc[i] = X + (size_t)m * K + g4 * 8;
    }
    const size_t WSTEP = PACKED ? (size_t)(N / 16) * 512 : 32;
    auto issue = [&](int step, int stage) {
        bf16* base = lds + (size_t)stage * BLKS * 512;
#pragma unroll
        for (int i = 0; i < WL; ++i)
            hb_load_to_lds(wsrc[i] + (size_t)step * WSTEP, base + (wave * WL + i) * 512);
#pragma unroll
        for (int i = 0; i < XL; ++i)
            hb_load_to_lds(xsrc[i] + (size_t)step * 32, base + (WBLK + wave * XL + i) * 512);
    };

    f32x16 acc[TN32][TM32];
#pragma unroll
    for (int a = 0; a < TN32; ++a)
#pragma unroll
        for (int b = 0; b < TM32; ++b)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[a][b][i] = 0.f;

    const int lane_off = (c32 >> 4) * 512 + (16 * g2 + (lane & 15)) * 8;   // + 32 * 8 for the second k-half
    bf16x8 wv[2][2][TN32], xv[2][2][TM32];       // [set][k-half][piece]
    auto read_operands = [&](int set, int stage) {
        const bf16* base = lds + (size_t)stage * BLKS * 512 + lane_off;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
#pragma unroll
            for (int a = 0; a < TN32; ++a)
                wv[set][h][a] = *(const bf16x8*)(base + (wn * TNB + 2 * a) * 512 + h * 256);
#pragma unroll
            for (int b = 0; b < TM32; ++b)
                xv[set][h][b] = *(const bf16x8*)(base + (WBLK + wm * TMB + 2 * b) * 512 + h * 256);
        }
    };
    auto multiply = [&](int set) {
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int a = 0; a < TN32; ++a)
#pragma unroll
                for (int b = 0; b < TM32; ++b)
                    acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wv[set][h][a], xv[set][h][b], acc[a][b],
                                                                        0, 0, 0);
    };
    // Before step t + 1 is read: this wave's loads of it have landed (those of the STAGES - 2 later
    // steps may be in flight) and its reads of step t are in registers; after the barrier that
    // holds for every wave, so the stage of step t can take the loads of step t + STAGES.
    auto advance = [&](int t) {
        hb_wait_vmcnt<(STAGES - 2) * (WL + XL)>();
        hb_workgroup_barrier();
        const int nt = t + STAGES;
        issue(nt < nsteps ? nt : nsteps - 1, nt % STAGES);
    };
    auto run_step = [&](int set, int t) {
        if (t + 1 < nsteps) {
            advance(t);
            read_operands(set ^ 1, (t + 1) % STAGES);
        }
        multiply(set);
    };
#pragma unroll
    for (int st = 0; st < STAGES - 1; ++st) issue(st < nsteps ? st : nsteps - 1, st);
    advance(-1);
    read_operands(0, 0);
    for (int t = 0; t < nsteps; t += 2) {
        run_step(0, t);
        if (t + 1 < nsteps) run_step(1, t + 1);
    }
    hb_wait_vmcnt<0>();      // the loads past the end (repeats of the last step) have landed too
    store_wave_tile<EPI, TN32, TM32>(acc, Cv, M, N, ldc, m0 + wm * TMB * 16, n0 + wn * TNB * 16, c32, g2);
}

// More than 64 KB of dynamic LDS has to be allowed per kernel, once.
static int allow_lds(const void* kernel, size_t lds) {
    static std::mutex lock;
    static std::unordered_set<const void*> allowed;
    std::lock_guard<std::mutex> guard(lock);
    if (allowed.count(kernel)) return 0;
    hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    HB_REQUIRE(e == hipSuccess, "gemm_mfma: cannot have %zu bytes of LDS: %s", lds, hipGetErrorString(e));
    allowed.insert(kernel);
    return 0;
}

template <class Kernel, class... Extra>
static int launch_tiles(Kernel kern, size_t lds, int threads, long total, int slices, const bf16* x, const bf16* w,
                        void* C, int M, int N, int K, int ldc, int m_tiles, int n_tiles, hipStream_t stream,
                        Extra... extra) {
    HB_REQUIRE(total < (1l << 30), "gemm_mfma: too many tiles");
    HB_REQUIRE(lds <= 160 * 1024, "gemm_mfma: %zu bytes of LDS asked for", lds);
    if (lds > 64 * 1024 && allow_lds((const void*)kern, lds) != 0) return 1;
    const dim3 blocks((unsigned)((total + 7) / 8 * 8), slices);
    kern<<<blocks, threads, lds, stream>>>(x, w, C, M, N, K, ldc, m_tiles, n_tiles, extra...);
    HB_CHECK_LAUNCH("gemm_tile");
    return 0;
}

#define TILE_DISPATCH(KERNEL, ...)                                                                   \
    do {                                                                                             \
        if (packed) {                                                                                \
            if (epi == EPI_STORE) return launch_tiles(KERNEL<EPI_STORE, true, __VA_ARGS__>, lds, threads, total, slices, x, w, C, M, N, K, ldc, m_tiles, n_tiles, stream EXTRA); \
            if (epi == EPI_ADD) return launch_tiles(KERNEL<EPI_ADD, true, __VA_ARGS__>, lds, threads, total, slices, x, w, C, M, N, K, ldc, m_tiles, n_tiles, stream EXTRA); \
            return launch_tiles(KERNEL<EPI_SWIGLU, true, __VA_ARGS__>, lds, threads, total, slices, x, w, C, M, N, K, ldc, m_tiles, n_tiles, stream EXTRA); \
        }                                                                                            \
        if (epi == EPI_STORE) return launch_tiles(KERNEL<EPI_STORE, false, __VA_ARGS__>, lds, threads, total, slices, x, w, C, M, N, K, ldc, m_tiles, n_tiles, stream EXTRA); \
        if (epi == EPI_ADD) return launch_tiles(KERNEL<EPI_ADD, false, __VA_ARGS__>, lds, threads, total, slices, x, w, C, M, N, K, ldc, m_tiles, n_tiles, stream EXTRA); \
        return launch_tiles(KERNEL<EPI_SWIGLU, false, __VA_ARGS__>, lds, threads, total, slices, x, w, C, M, N, K, ldc, m_tiles, n_tiles, stream EXTRA); \
    } while (0)

// slices > 1: the sums of the slices go to `partial`; the caller adds them up afterwards
template <int TNB, int TMB, int WNW, int WMW, int WST, int XST>
static int launch_tile64(const void* X, const void* W, void* C, int M, int N, int K, int ldc, int epi, int packed,
                         hipStream_t stream, int slices = 1, float* partial = nullptr, RowScale scale = RowScale{}) {
    constexpr int BN = 16 * TNB * WNW, BM = 16 * TMB * WMW;
    HB_REQUIRE(K % 64 == 0, "gemm_mfma: K=%d is no multiple of 64", K);
    const int m_tiles = (M + BM - 1) / BM, n_tiles = (N + BN - 1) / BN;
    const long total = (long)m_tiles * n_tiles;
    const size_t lds = (size_t)(WST * BN + XST * BM) * 64 * sizeof(bf16) + WNW * WMW * 16 * sizeof(float);
    const int threads = 64 * WNW * WMW;
    const bf16* x = (const bf16*)X;
    const bf16* w = (const bf16*)W;
    HB_REQUIRE(slices >= 1 && (slices == 1 || partial), "gemm_mfma: bad slices");
    // (a handed-on norm and K slices go together: every slice's sums are scaled, and so is their sum)
    HB_REQUIRE(!scale.partial || (M <= 16 && epi != EPI_ADD), "gemm_mfma: this product takes no handed-on norm");
    HB_REQUIRE((K / 64 + slices - 1) / slices * (slices - 1) < K / 64, "gemm_mfma: a slice of K would be empty");
#define EXTRA , partial, QkvEpilogue{}, scale
    TILE_DISPATCH(gemm_tile_kernel, TNB, TMB, WNW, WMW, WST, XST);
#undef EXTRA
}

// Tiles whose width is no power of two (192 = three pieces of 32 a wave): for the SwiGLU epilogue
// only, whose bfloat16 output goes to memory lane by lane (the float32 epilogues' way through LDS
// counts on rows of a power of two of 16-byte chunks).
template <int TNB, int TMB, int WNW, int WMW, int WST, int XST>
static int launch_tile64_swiglu(const void* X, const void* W, void* C, int M, int N, int K, int ldc, int epi,
                                int packed, hipStream_t stream, int slices) {
    constexpr int BN = 16 * TNB * WNW, BM = 16 * TMB * WMW;
    HB_REQUIRE(epi == EPI_SWIGLU && slices == 1, "gemm_mfma: this tile takes the SwiGLU product whole only");
    HB_REQUIRE(K % 64 == 0, "gemm_mfma: K=%d is no multiple of 64", K);
    const int m_tiles = (M + BM - 1) / BM, n_tiles = (N + BN - 1) / BN;
    const long total = (long)m_tiles * n_tiles;
    const size_t lds = (size_t)(WST * BN + XST * BM) * 64 * sizeof(bf16) + WNW * WMW * 16 * sizeof(float);
    const bf16* x = (const bf16*)X;
    const bf16* w = (const bf16*)W;
    if (packed)
        return launch_tiles(gemm_tile_kernel<EPI_SWIGLU, true, TNB, TMB, WNW, WMW, WST, XST>, lds, 64 * WNW * WMW, total, 1,
                            x, w, C, M, N, K, ldc, m_tiles, n_tiles, stream, (float*)nullptr, QkvEpilogue{}, RowScale{});
    return launch_tiles(gemm_tile_kernel<EPI_SWIGLU, false, TNB, TMB, WNW, WMW, WST, XST>, lds, 64 * WNW * WMW, total, 1,
                        x, w, C, M, N, K, ldc, m_tiles, n_tiles, stream, (float*)nullptr, QkvEpilogue{}, RowScale{});
}

template <int TNB, int TMB, int WNW, int WMW, int STAGES>
static int launch_tile32(const void* X, const void* W, void* C, int M, int N, int K, int ldc, int epi, int packed,
                         hipStream_t stream) {
    constexpr int BN = 16 * TNB * WNW, BM = 16 * TMB * WMW;
    const int m_tiles = (M + BM - 1) / BM, n_tiles = (N + BN - 1) / BN;
    const long total = (long)m_tiles * n_tiles;
    const size_t lds = (size_t)STAGES * (BN + BM) * 32 * sizeof(bf16);
    const int threads = 64 * WNW * WMW;
    const bf16* x = (const bf16*)X;
    const bf16* w = (const bf16*)W;
    const int slices = 1;
#define EXTRA
    TILE_DISPATCH(gemm_tile32_kernel, TNB, TMB, WNW, WMW, STAGES);
#undef EXTRA
}
#undef TILE_DISPATCH

// The q/k/v projection of a step with many rows, fused with norm, rotation and cache write
// (see QkvEpilogue). X [M, K] bf16; W [(nq + 2 nkv) 128, K] bf16, rows q | k | v. A wave's tile is
// one head wide; shape: 0 = tiles of 256 x 256 (waves 2 x 2, for long prompts), 1 = a head wide and 256
// rows high (four waves one above the other, 64 rows each), 2 = a head wide and 128 rows high (32
// rows a wave): more and smaller tiles for prompts whose 256 x 256 tiles would not fill the CUs.
template <int TNB, int TMB, int WNW, int WMW, int WST, int XST>
static int launch_qkv(const bf16* x, const bf16* w, int M, int N, int K, int packed, const QkvEpilogue& e,
                      hipStream_t stream) {
    constexpr int BN = 16 * TNB * WNW, BM = 16 * TMB * WMW;
    const int m_tiles = (M + BM - 1) / BM, n_tiles = (N + BN - 1) / BN;
    const long total = (long)m_tiles * n_tiles;
    const size_t lds = (size_t)(WST * BN + XST * BM) * 64 * sizeof(bf16) + WNW * WMW * 16 * sizeof(float);
    if (packed)
        return launch_tiles(gemm_tile_kernel<EPI_QKV, true, TNB, TMB, WNW, WMW, WST, XST>, lds, 64 * WNW * WMW, total, 1, x,
                            w, nullptr, M, N, K, N, m_tiles, n_tiles, stream, (float*)nullptr, e, RowScale{});
    return launch_tiles(gemm_tile_kernel<EPI_QKV, false, TNB, TMB, WNW, WMW, WST, XST>, lds, 64 * WNW * WMW, total, 1, x, w,
                        nullptr, M, N, K, N, m_tiles, n_tiles, stream, (float*)nullptr, e, RowScale{});
}

extern "C" int hb_gemm_qkv_mfma(const void* X, const void* W, int M, int K, int packed, void* q_out, void* k_cache,
                                void* v_cache, const int* positions, const int* seq_of, const int* slots,
                                const int* page_table, int max_pages, int page_size, const float* q_norm_w,
                                const float* k_norm_w, const float* cos_t, const float* sin_t, float eps, int nq,
                                int nkv, int hd, int shape, hipStream_t stream) {
    HB_REQUIRE(hd == 128 && page_size == 64, "gemm_qkv: heads of 128 and pages of 64 tokens only");
    HB_REQUIRE(M > 0 && nq > 0 && nkv > 0 && K > 0 && K % 64 == 0, "gemm_qkv: bad sizes (M=%d, K=%d)", M, K);
    HB_REQUIRE((cos_t == nullptr) == (sin_t == nullptr), "gemm_qkv: cos and sin tables come together");
    HB_REQUIRE(shape >= 0 && shape <= 2, "gemm_qkv: unknown tile shape %d", shape);
    const int N = (nq + 2 * nkv) * 128;
    const QkvEpilogue e = {(bf16*)q_out, (bf16*)k_cache, (bf16*)v_cache, positions, seq_of, slots, page_table,
                           max_pages, q_norm_w, k_norm_w, cos_t, sin_t, eps, nq, nkv};
    const bf16* x = (const bf16*)X;
    const bf16* w = (const bf16*)W;
    if (shape == 0) return launch_qkv<8, 8, 2, 2, 2, 2>(x, w, M, N, K, packed, e, stream);
    if (shape == 1) return launch_qkv<8, 4, 1, 4, 3, 2>(x, w, M, N, K, packed, e, stream);
    return launch_qkv<8, 2, 1, 4, 3, 2>(x, w, M, N, K, packed, e, stream);
}

// Which kernel a product runs on: tile 0 = the few-row kernel, otherwise a tile variant by number and
// the number of K slices; tile -1: nothing takes this product with what is asked of it. The flags
// say whether the input is normed on the way (norm_w), a norm is left behind (emit_g) or a handed-on
// one is finished (scale_partial).
struct GemmPlan { int tile, slices; double cost = -1; };      // cost: the estimated time in us where the plan was chosen by one
static GemmPlan plan_gemm(int M, int N, int K, int ldc, int epi, bool norm_w, bool emit_g, bool scale_partial,
                          int tile_hint, size_t workspace_floats, bool deferred = false) {
    int tile = tile_hint % 1000, slices = tile_hint >= 1000 ? tile_hint / 1000 : 1;
    double low_cost = -1, mid_cost = -1;
    if (tile_hint == 1) return M <= 16 ? GemmPlan{0, 1} : GemmPlan{-1, 0};      // the few-row kernel, asked for by name
    // no slice of K may be empty, and each has at least four steps to run through its ring
    auto slices_fit = [&](int steps, int sl) {
        const int per = (steps + sl - 1) / sl;
        return steps / sl >= 4 && per * (sl - 1) < steps && (size_t)sl * M * N <= workspace_floats;
    };
    // What the second kernel of a product cut into slices can leave behind: rows of at most 8192.
    const bool reducer_norms = N % 4 == 0 && N <= 8192 && ldc % 4 == 0;
    if (tile == 0 && M <= 64) {
        // At most 64 rows: the product is bound by the weights it reads, and what counts is how
        // evenly and how deeply the CUs stream them. Candidates: the few-row kernel (at most 16
        // rows; its waves take the weights from HBM straight into their MFMA operands) and the tiled
        // kernel with tiles one block of rows high and K cut into 1 to 16 slices. Taken: the least
        // estimated time (us). The estimates were fitted to measurements of the four products of a
        // layer for six model sizes (hidden 1024 to 5120) and 4 to 64 rows; the choice is within 1 %
        // of the best candidate on average and within 12 % at worst.
        double best = -1;
        bool skinny = false;
        if (M <= 16) {
            // Workgroups of 16 (or 64) weight rows, each streaming at a rate of its own: about
            // 24 KB/us alone on a CU (more if some CUs stay empty), 28 KB/us for a CU with several of 16 rows;
            // more rows cost more reads of the activations. 320 workgroups on 256 CUs take as long as 512.
            const int nb = (epi == EPI_SWIGLU || N >= 16384) ? 4 : 1;
            const long wgs = (N + 16 * nb - 1) / (16 * nb);
            const double rounds = wgs <= 256 ? 1 : (wgs <= 512 ? 2 : wgs / 256.0 + 0.5);
            double rate = (wgs <= 256 || nb == 4 ? 24e3 : 28e3) / (1 + 0.02 * M);
            if (wgs < 256) rate *= 1 + 0.6 * (256 - wgs) / 256.0;
            best = 3.0 + rounds * 32.0 * nb * K / rate;
            skinny = true;
        }
        if (!norm_w && K % 64 == 0) {
            struct Small { int id, bn, bm, per_cu; double step_us; };
            // (164: tiles of 96 columns for the SwiGLU product of 33 to 64 rows, whole: 256 of them where
            // tiles of 128 are 192, e.g. 24576 x 4096 at 64 rows 43 -> 40 us, 19456 x 2560 29 -> 26 us;
            // for fewer rows the tile of 32 rows stays ahead)
            static const Small small[] = {{112, 128, 32, 2, 0.5}, {124, 128, 64, 2, 0.6}, {184, 256, 64, 1, 0.9},
                                          {164, 96, 64, 2, 0.585}};
            const int steps = K / 64;
            for (const Small& v : small) {
                if (M > v.bm) continue;
                if (scale_partial && v.id != 112) continue;            // only this one finishes a handed-on norm
                if (v.id == 164 && (epi != EPI_SWIGLU || M <= 32)) continue;
                const long tiles = (N + v.bn - 1) / v.bn;
                for (int sl = 1; sl <= 16; sl *= 2) {
                    if (sl > 1 && (v.id == 164 || !slices_fit(steps, sl))) break;
                    // a norm is left behind by the kernel that adds the slices up
                    if (emit_g && (sl == 1 || !reducer_norms)) continue;
                    if (deferred && sl > 8) break;                 // whoever adds the slices up takes 2, 4 or 8
                    const long wgs = tiles * sl, slots = 256 * v.per_cu;
                    const long rounds = (wgs + slots - 1) / slots;
                    const long on_a_cu = ((wgs < slots ? wgs : slots) + 255) / 256;
                    const int per = (steps + sl - 1) / sl;
                    const double waiting = (double)rounds * per * v.step_us * on_a_cu;       // bound by latency
                    double streaming = (double)wgs * per * (v.bn * 128 + v.bm * 64) / 6.0e6;   // bound by HBM
                    if (v.id == 164) streaming /= 1.2;         // (a round of 256 workgroups streams a fifth faster than one of 192)
                    if (wgs > slots) streaming *= 1.12;
                    double cost = (waiting > streaming ? waiting : streaming) + 3.0;
                    if (sl > 1) cost += deferred ? 0.3 * sl : 2.5 + (double)(sl + 1) * M * N * 4 / 2.0e6 + (emit_g ? 1.5 : 0.0);
                    if (best < 0 || cost < best) {
                        best = cost;
                        skinny = false;
                        tile = v.id;
                        slices = sl;
                    }
                }
            }
        }
        if (skinny) return GemmPlan{0, 1, best};
        low_cost = best;
        if (tile == 0) {
            if (emit_g || scale_partial) return GemmPlan{-1, 0};
            tile = 123;
        }
    }
    if (norm_w) return GemmPlan{-1, 0};
    if (tile == 0 && K % 64) tile = 123;
    if (tile == 0 && K % 64 == 0) {
        // More than 64 rows: neither the arithmetic nor the weights alone decide. All tiles from 128 x 64
        // to 256 x 256 with 1 to 16 K slices are candidates; a candidate takes as long as the slowest
        // of: its workgroups' steps one after another (a step's time alone on a CU, about twice that
        // with two on a CU), what all workgroups move out of the L2s (16 TB/s), what comes from
        // HBM once (7 TB/s); plus a start and, for slices, the second kernel. Fitted to the four
        // products of a layer for three model sizes and 96 to 1024 rows (the choice is then 1 % from
        // the best candidate on average, 12 % at worst), checked on three other sizes (2 %, 13 %) and
        // on 1280 to 4096 rows (under 1 %, 7 %).
        struct Mid { int id, bn, bm, per_cu; double step_us; };
        // (168: three quarters of the 256 x 256 tile's arithmetic a step, for the SwiGLU product whole:
        // where that one's tiles fill the last round of 256 badly, 192 columns often fill it)
        // (186: 192 rows high, for row counts whose tiles of 256 rows leave CUs empty and whose tiles of
        // 128 rows need a second round: 2,400 to 3,072 rows of 4096 columns, 6 to 14 % off)
        static const Mid mid[] = {{188, 256, 256, 1, 1.26}, {142, 256, 128, 1, 0.77}, {122, 128, 128, 2, 0.95},
                                  {124, 128, 64, 2, 0.48}, {184, 256, 64, 1, 0.67}, {168, 192, 256, 1, 1.0},
                                  {186, 256, 192, 1, 1.08}};
        const int steps = K / 64;
        double best = -1;
        for (const Mid& v : mid) {
            if (v.id == 168 && epi != EPI_SWIGLU) continue;
            const long tiles = (long)((M + v.bm - 1) / v.bm) * ((N + v.bn - 1) / v.bn);
            for (int sl = 1; sl <= 16; sl *= 2) {
                if (v.id == 168 && sl > 1) break;
                if (sl > 1 && !slices_fit(steps, sl)) break;
                if (emit_g && (sl == 1 || !reducer_norms)) continue;      // the kernel that adds the slices up norms
                if (deferred && sl > 8) break;                            // whoever adds the slices up takes 2, 4 or 8
                const long wgs = tiles * sl, slots = 256 * v.per_cu;
                const long rounds = (wgs + slots - 1) / slots;
                const long on_a_cu = ((wgs < slots ? wgs : slots) + 255) / 256;
                const int per = (steps + sl - 1) / sl;
                const double stepping = (double)rounds * per * v.step_us * (1 + 1.06 * (on_a_cu - 1));
                const double moving = (double)wgs * per * (v.bn + v.bm) * 128 / 16.3e6;
                const double fetching = ((double)N + M) * K * 2 / 7.1e6;
                double cost = stepping > moving ? stepping : moving;
                if (fetching > cost) cost = fetching;
                cost += 2.3;
                if (sl > 1) cost += deferred ? (double)sl * M * N * 4 / 2.3e6 : 1.5 + (double)(sl + 1) * M * N * 4 / 2.3e6;
                if (best < 0 || cost < best) {
                    best = cost;
                    tile = v.id;
                    slices = sl;
                }
            }
        }
        mid_cost = best;
    }
    // (tile_hint: 0 = choose; otherwise a variant by number, for measurements and tests, + 1000 x
    // the number of K slices; 1 = the few-row kernel)
    if (emit_g && !(slices > 1 && reducer_norms)) return GemmPlan{-1, 0};
    return GemmPlan{tile, slices, mid_cost >= 0 ? mid_cost : low_cost};
}

// The rows of the first of two products that M rows are better cut into (see hb_gemm_mfma), or 0.
static int split_rows(int M, int N, int K, int ldc, int epi, bool special, int tile_hint, size_t workspace_floats,
                      const GemmPlan& whole) {
    if (special || M <= 128 || (tile_hint != 0 && tile_hint != -128 && tile_hint != -256)) return 0;
    int best_main = 0;
    double best = whole.cost;
    for (int bm = 128; bm <= 256; bm *= 2) {
        const int main_rows = M / bm * bm, rest = M - main_rows;
        if (rest == 0 || main_rows == 0) continue;
        const GemmPlan a = plan_gemm(main_rows, N, K, ldc, epi, false, false, false, 0, workspace_floats);
        const GemmPlan b = plan_gemm(rest, N, K, ldc, epi, false, false, false, 0, workspace_floats);
        if (a.tile < 0 || b.tile < 0) continue;
        if (tile_hint == -bm) return main_rows;
        if (tile_hint != 0 || whole.cost < 0 || a.cost < 0 || b.cost < 0) continue;
        // (a second launch and its start are in the estimates; a tenth is kept as a margin for their error)
        if (a.cost + b.cost < 0.9 * best) {
            best = (a.cost + b.cost) / 0.9;
            best_main = main_rows;
        }
    }
    return best_main;
}

// The rows that hb_gemm_mfma cuts off as a first product of their own, or 0 (for tests and measurements).
extern "C" int hb_gemm_mfma_split(int M, int N, int K, int epi, size_t workspace_floats) {
    const int ldc = epi == EPI_SWIGLU ? N / 2 : N;
    const GemmPlan whole = plan_gemm(M, N, K, ldc, epi, false, false, false, 0, workspace_floats);
    return whole.tile < 0 ? 0 : split_rows(M, N, K, ldc, epi, false, 0, workspace_floats, whole);
}

// The plan as a number for tests and measurements: tile + 1000 x slices (slices > 1), 0 for the
// few-row kernel, -1 if the product is refused. emit: 0 none, 1 a norm is left behind. deferred:
// the slices are left for the next kernel to add up.
extern "C" int hb_gemm_mfma_plan(int M, int N, int K, int epi, int normed_input, int emit, int scaled,
                                 size_t workspace_floats, int deferred) {
    const GemmPlan p = plan_gemm(M, N, K, epi == EPI_SWIGLU ? N / 2 : N, epi, normed_input != 0, emit != 0, scaled != 0, 0,
                                 workspace_floats, deferred != 0);
    return p.tile <= 0 ? p.tile : p.tile + (p.slices > 1 ? 1000 * p.slices : 0);
}

// The estimated time in us of the plan that hb_gemm_mfma_plan gives, or a negative number where the
// plan is not chosen by an estimate (the few products that only one kernel takes).
extern "C" double hb_gemm_mfma_plan_cost(int M, int N, int K, int epi, int normed_input, int emit, int scaled,
                                         size_t workspace_floats, int deferred) {
    return plan_gemm(M, N, K, epi == EPI_SWIGLU ? N / 2 : N, epi, normed_input != 0, emit != 0, scaled != 0, 0,
                     workspace_floats, deferred != 0).cost;
}

// C (+)= X @ W^T. X [M, K] bf16, W [N, K] bf16. epi 0: C f32 [M, N] stored; 1: added to;
// 2: W's rows are gate/up interleaved in blocks of 16 and C is bf16 [M, N / 2] = silu(gate) * up.
// packed != 0: W is stored as [K / 32][N / 16][64 lanes][8]: lane = 16 * (k / 8 % 4) + n % 16.
// All blocks of one k-step lie together: workgroups that advance through K side by side read one
// contiguous stretch of memory at a time, as a streaming copy would.
// workspace: float scratch for K cut into slices (more than 16 rows); without it K is not cut.
// norm_w != null: X is the float32 residual stream [M, K] and the product is RMSNorm(X; norm_w, eps) W^T
// (M <= 16 only, never with the add epilogue).
// emit_*, scale_*: see NormHandoff (all null / 0 for a product that neither leaves nor takes a norm).
extern "C" int hb_gemm_mfma(const void* X, const void* W, void* C, int M, int N, int K, int ldc, int epi,
                            int packed, const float* norm_w, float eps, int tile_hint, float* workspace,
                            size_t workspace_floats, const float* emit_g, void* emit_xg, float* emit_partial,
                            const float* scale_partial, int scale_parts, float scale_eps, float emit_eps,
                            int* deferred_slices, hipStream_t stream) {
    const NormHandoff hand = {emit_g, (bf16*)emit_xg, emit_partial, scale_partial, scale_parts, scale_eps, emit_eps};
    const bool emit_whole = emit_g && !emit_partial;      // the second kernel of a product cut into slices norms
    HB_REQUIRE(!scale_partial || (M <= 16 && !norm_w), "gemm_mfma: a norm is handed on for at most 16 rows");
    HB_REQUIRE(!emit_g || (epi == EPI_ADD && emit_xg && !norm_w), "gemm_mfma: only the adding product leaves a norm behind");
    HB_REQUIRE(!emit_g || (emit_whole ? M > 16 : M <= 16),
               "gemm_mfma: a norm is left half done for at most 16 rows, whole for more");
    HB_REQUIRE(!scale_partial || (scale_parts > 0 && epi != EPI_ADD), "gemm_mfma: bad partial sums of a handed-on norm");
    HB_REQUIRE(!norm_w || (M <= 16 && epi != EPI_ADD && (epi == EPI_SWIGLU || N >= 16384)),
               "gemm_mfma: the fused norm takes M <= 16, N >= 16384 and no add");
    HB_REQUIRE(!packed || N % 16 == 0, "gemm_mfma: packed weights need N %% 16 == 0");
    HB_REQUIRE(M > 0 && N > 0 && K > 0, "gemm_mfma: empty problem (M=%d, N=%d, K=%d)", M, N, K);
    HB_REQUIRE(epi >= 0 && epi <= 2, "gemm_mfma: unknown epilogue %d", epi);
    HB_REQUIRE(K % 32 == 0, "gemm_mfma: K=%d is no multiple of 32", K);
    HB_REQUIRE(epi != EPI_SWIGLU || N % 32 == 0, "gemm_mfma: the SwiGLU epilogue needs N %% 32 == 0");
    HB_REQUIRE(ldc >= (epi == EPI_SWIGLU ? N / 2 : N), "gemm_mfma: output row stride %d too small", ldc);
    const RowScale row_scale = {scale_partial, scale_parts, scale_eps};
    // deferred_slices != null (plain store only): if K is cut into slices, they are left in the
    // workspace [slice][M][N] for the caller's next kernel to add up, and their number is written
    // there; 1 means C holds the product as usual.
    HB_REQUIRE(!deferred_slices || (epi == EPI_STORE && !emit_g), "gemm_mfma: only a plain product leaves its slices");
    if (deferred_slices) *deferred_slices = 1;
    const GemmPlan plan = plan_gemm(M, N, K, ldc, epi, norm_w != nullptr, emit_g != nullptr, scale_partial != nullptr,
                                    tile_hint < 0 ? 0 : tile_hint, workspace_floats, deferred_slices != nullptr);
    HB_REQUIRE(plan.tile >= 0, "gemm_mfma: no kernel takes M=%d, N=%d, K=%d with the norm asked of it", M, N, K);
    // Rows that end a little past a whole number of tiles pay a round of tiles for a few rows (a
    // prompt of 2,049 tokens took a quarter longer than one of 2,048). Such a product is cut in
    // two along its rows, the whole tiles and the rest as products of their own (the epilogues
    // work row by row), where the estimates say that this is a good deal faster.
    // tile_hint -128 / -256: cut there whatever the estimates say (for tests).
    const int rows_main = split_rows(M, N, K, ldc, epi, norm_w || emit_g || scale_partial || deferred_slices, tile_hint,
                                     workspace_floats, plan);
    if (rows_main > 0) {
        const size_t out_bytes = epi == EPI_SWIGLU ? sizeof(bf16) : sizeof(float);
        const int rc = hb_gemm_mfma(X, W, C, rows_main, N, K, ldc, epi, packed, nullptr, eps, 0, workspace, workspace_floats,
                                    nullptr, nullptr, nullptr, nullptr, 0, 0.f, 0.f, nullptr, stream);
        if (rc != 0) return rc;
        return hb_gemm_mfma((const bf16*)X + (size_t)rows_main * K, W, (char*)C + (size_t)rows_main * ldc * out_bytes,
                            M - rows_main, N, K, ldc, epi, packed, nullptr, eps, 0, workspace, workspace_floats, nullptr,
                            nullptr, nullptr, nullptr, 0, 0.f, 0.f, nullptr, stream);
    }
    if (plan.tile == 0) {
        pick_skinny(X, W, C, M, N, K, ldc, epi, packed, norm_w, eps, stream, hand);
        HB_CHECK_LAUNCH("gemm_skinny");
        return 0;
    }
    const int tile = plan.tile, slices = plan.slices;
    HB_REQUIRE(slices == 1 || (size_t)slices * M * N <= workspace_floats, "gemm_mfma: no room for %d slices", slices);
    HB_REQUIRE(!scale_partial || tile == 112, "gemm_mfma: only the few-row kernels take a handed-on norm");
    int rc;
    switch (tile) {
        // (ring depths, measured with weights that come from HBM: a third weight stage gains a
        // tenth for 256 x 128 and nothing for the other two; a third activation stage nothing)
        case 188: rc = launch_tile64<8, 8, 2, 2, 2, 2>(X, W, C, M, N, K, ldc, epi, packed, stream, slices, workspace); break;   // 256 x 256
        case 142: rc = launch_tile64<8, 4, 2, 2, 3, 2>(X, W, C, M, N, K, ldc, epi, packed, stream, slices, workspace); break;   // 256 (n) x 128 (m)
        case 186: rc = launch_tile64<8, 6, 2, 2, 2, 2>(X, W, C, M, N, K, ldc, epi, packed, stream, slices, workspace); break;   // 256 (n) x 192 (m)
        case 122: rc = launch_tile64<4, 4, 2, 2, 2, 2>(X, W, C, M, N, K, ldc, epi, packed, stream, slices, workspace); break;   // 128 x 128, two to a CU
        case 124: rc = launch_tile64<2, 4, 4, 1, 3, 2>(X, W, C, M, N, K, ldc, epi, packed, stream, slices, workspace); break;   // 128 (n) x 64 (m)
        case 112: rc = launch_tile64<2, 2, 4, 1, 3, 2>(X, W, C, M, N, K, ldc, epi, packed, stream, slices, workspace, row_scale); break;   // 128 (n) x 32 (m)
        case 184: rc = launch_tile64<4, 4, 4, 1, 3, 2>(X, W, C, M, N, K, ldc, epi, packed, stream, slices, workspace); break;   // 256 (n) x 64 (m)
        case 168: rc = launch_tile64_swiglu<6, 8, 2, 2, 2, 2>(X, W, C, M, N, K, ldc, epi, packed, stream, slices); break;   // 192 (n) x 256 (m)
        case 164: rc = launch_tile64_swiglu<6, 2, 1, 2, 3, 2>(X, W, C, M, N, K, ldc, epi, packed, stream, slices); break;   // 96 (n) x 64 (m), two waves one above the other
        case 123:                                                                                                           // 128 x 128, K in steps of 32
            HB_REQUIRE(slices == 1, "gemm_mfma: this tile does not cut K");
            return launch_tile32<4, 4, 2, 2, 4>(X, W, C, M, N, K, ldc, epi, packed, stream);
        default: HB_REQUIRE(false, "gemm_mfma: unknown tile %d", tile);
    }
    if (rc == 0 && slices > 1 && deferred_slices) {
        *deferred_slices = slices;
        return 0;
    }
    if (rc == 0 && slices > 1) {
        const size_t total = (size_t)M * N;
        if (emit_g)
            if (M <= 64)
                gemm_slices_norm_kernel<1024, 2, 8><<<M, 1024, 0, stream>>>(workspace, (float*)C, M, N, ldc, slices, emit_g,
                                                                             emit_eps, (bf16*)emit_xg, emit_partial);
            else if (N <= 4096)   // many rows: smaller blocks, several to a CU, that hide each other's waits
                gemm_slices_norm_kernel<256, 4, 2><<<M, 256, 0, stream>>>(workspace, (float*)C, M, N, ldc, slices, emit_g,
                                                                           emit_eps, (bf16*)emit_xg, emit_partial);
            else
                gemm_slices_norm_kernel<256, 8, 2><<<M, 256, 0, stream>>>(workspace, (float*)C, M, N, ldc, slices, emit_g,
                                                                           emit_eps, (bf16*)emit_xg, emit_partial);
        else if (epi == EPI_SWIGLU)
            gemm_slices_swiglu_kernel<<<(unsigned)((total / 2 + 255) / 256), 256, 0, stream>>>(workspace, (bf16*)C, M, N,
                                                                                             ldc, slices);
        else
            gemm_slices_kernel<<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(workspace, (float*)C, M, N, ldc,
                                                                                  slices, epi == EPI_ADD);
        HB_CHECK_LAUNCH("gemm_slices");
    }
    return rc;
}
