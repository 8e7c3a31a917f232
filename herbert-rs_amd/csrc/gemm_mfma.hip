// bfloat16 matrix products on the gfx950 matrix cores, float32 accumulation:
//   C[m, n] (+)= sum_k X[m, k] * W[n, k]        X [M, K], W [N, K], both k-contiguous
// Two kernels share the epilogues:
//   skinny (M <= 64, decoding): HBM-bound. The weights stream from memory straight into
//     MFMA operands (each is used once), four waves of a workgroup split K between them
//     and add their parts through LDS in a fixed order.
//   tiled (M > 64, prompts): 256 x 256 or 128 x 128 tiles loaded from global memory straight
//     into a ring of LDS stages, one or two k-steps ahead of the MFMAs that consume them.
// In both the weight rows are the MFMA's first operand, so a lane ends up with four
// consecutive n of one m: row-major stores of C are vector stores.
// Epilogues: 0 store float32, 1 add to float32 (the residual stream), 2 SwiGLU to bfloat16
// (weight rows interleaved in blocks of 16: gate rows, then the up rows of the same outputs).
#include "common.h"

HB_MODULE_ERROR_SLOT()

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

#define EPI_STORE 0
#define EPI_ADD 1
#define EPI_SWIGLU 2

__device__ __forceinline__ float silu_mul(float g, float u) { return g / (1.0f + __expf(-g)) * u; }

// ------------------------------------------------------------------ skinny
// Workgroup: WAVES waves, NB blocks of 16 weight rows, MB blocks of 16 activation rows.
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

template <int MB, int NB, int WAVES, int EPI, bool PACKED, bool NORM>
__global__ void __launch_bounds__(WAVES * 64)
gemm_skinny_kernel(const void* __restrict__ Xv, const bf16* __restrict__ W, void* __restrict__ Cv, int M,
                   int N, int K, int ldc, const float* __restrict__ norm_w, float eps,
                   float* __restrict__ partial) {
    constexpr int U = NORM ? 2 : ((NB + MB <= 4) ? 4 : 2);
    const bf16* X = (const bf16*)Xv;
    const float* XF = (const float*)Xv;
    extern __shared__ float red[];   // [WAVES / 2][NB * MB * 4][64]
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int r16 = lane & 15;
    const int g4 = lane >> 4;
    const int n0 = blockIdx.x * (NB * 16);
    const int k32 = K / 32;                       // k-steps of the whole product
    // gridDim.y > 1: this workgroup sums one slice of K only and leaves its sums in `partial`
    // [slice][M][N]; a second kernel adds the slices in order (see gemm_slices_kernel)
    const int per_slice = (k32 + gridDim.y - 1) / gridDim.y;
    const int step0 = blockIdx.y * per_slice;
    const int nsteps = k32 - step0 < per_slice ? (k32 - step0 > 0 ? k32 - step0 : 0) : per_slice;

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

    const int mine = wave < nsteps ? (nsteps - wave + WAVES - 1) / WAVES : 0;   // this wave's steps
    const int groups = mine / U;
    SkinnyOperands<MB, NB, NORM> cur[U], nxt[U];

#define SKINNY_LOAD(dst, group)                                                  \
    _Pragma("unroll") for (int u = 0; u < U; ++u) {                              \
        const int st = step0 + wave + ((group) * U + u) * WAVES;                 \
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
    for (int g = 0; g < groups; g += 2) {
        if (g + 1 < groups) { SKINNY_LOAD(nxt, g + 1) }
        SKINNY_MULTIPLY(cur)
        if (g + 1 < groups) {
            if (g + 2 < groups) { SKINNY_LOAD(cur, g + 2) }
            SKINNY_MULTIPLY(nxt)
        }
    }
    for (int i = groups * U; i < mine; ++i) {       // what is left over of this wave's steps
        const int st = step0 + wave + i * WAVES;
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

    // lane: m = b * 16 + r16, n = n0 + a * 16 + g4 * 4 + i
    if (gridDim.y > 1) {
        float* P = partial + (size_t)blockIdx.y * M * N;
#pragma unroll
        for (int a = 0; a < NB; ++a)
#pragma unroll
            for (int b = 0; b < MB; ++b) {
                const int m = b * 16 + r16;
                if (m >= M) continue;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int n = n0 + a * 16 + g4 * 4 + i;
                    if (n < N) P[(size_t)m * N + n] = acc[a][b][i];
                }
            }
        return;
    }
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
#pragma unroll
        for (int a = 0; a < NB; ++a)
#pragma unroll
            for (int b = 0; b < MB; ++b) {
                const int m = b * 16 + r16;
                if (m >= M) continue;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int n = n0 + a * 16 + g4 * 4 + i;
                    if (n < N) {
                        const size_t idx = (size_t)m * ldc + n;
                        if (EPI == EPI_ADD)
                            C[idx] += acc[a][b][i];
                        else
                            C[idx] = acc[a][b][i];
                    }
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

template <int MB, int NB, int WAVES>
static void launch_skinny(const void* X, const void* W, void* C, int M, int N, int K, int ldc, int epi,
                          int packed, const float* norm_w, float eps, hipStream_t stream,
                          float* partial = nullptr, int slices = 1) {
    const dim3 blocks((N + NB * 16 - 1) / (NB * 16), slices);
    size_t lds = (size_t)(WAVES / 2) * NB * MB * 4 * 64 * sizeof(float);
    if (lds < (size_t)WAVES * MB * 16 * sizeof(float)) lds = (size_t)WAVES * MB * 16 * sizeof(float);
    const bf16* w = (const bf16*)W;
#define SKINNY_GO(EPIV, PK, NM)                                                                        \
    gemm_skinny_kernel<MB, NB, WAVES, EPIV, PK, NM><<<blocks, WAVES * 64, lds, stream>>>(X, w, C, M, N, K, \
                                                                                          ldc, norm_w, eps, partial)
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
    if (slices > 1) {
        const size_t total = (size_t)M * N;
        gemm_slices_kernel<<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(partial, (float*)C, M, N, ldc, slices,
                                                                              epi == EPI_ADD);
    }
}

template <int MB>
static void pick_skinny(const void* X, const void* W, void* C, int M, int N, int K, int ldc, int epi,
                        int packed, const float* norm_w, float eps, hipStream_t stream, float* workspace,
                        size_t workspace_floats) {
    if (MB >= 2 && !norm_w) {
        // More than 16 rows: every workgroup re-reads its slice of the activations from L2, so a
        // workgroup takes 64 weight rows (the activations are then read as often as the weights),
        // and K is cut into slices over further workgroups until the 256 CUs have work; the slices'
        // sums are added in order by a second kernel, so the result does not depend on timing.
        const int groups = (N + 63) / 64;
        int slices = 1;
        if (epi != EPI_SWIGLU) {
            slices = 256 / groups;
            const int most = K / 32 / 8;                 // at least one k-step a wave
            if (slices > most) slices = most;
            if (slices > 8) slices = 8;
            if (slices < 1) slices = 1;
            if ((size_t)slices * M * N > workspace_floats) slices = 1;
        }
        if (slices == 1 && N >= 16384)      // wide enough without slices: four waves a workgroup, more of them a CU
            launch_skinny<MB, 4, 4>(X, W, C, M, N, K, ldc, epi, packed, norm_w, eps, stream);
        else
            launch_skinny<MB, 4, 8>(X, W, C, M, N, K, ldc, epi, packed, norm_w, eps, stream, workspace, slices);
        return;
    }
    // Few weight rows: one block of 16 rows a workgroup and eight waves splitting K, so that the
    // 256 CUs all have work. Many rows: more rows a workgroup, so that the activations are
    // re-read from L2 less often.
    if (epi == EPI_SWIGLU || N >= 16384) {
        launch_skinny<MB, 4, 4>(X, W, C, M, N, K, ldc, epi, packed, norm_w, eps, stream);
    } else {
        launch_skinny<MB, 1, 8>(X, W, C, M, N, K, ldc, epi, packed, norm_w, eps, stream);
    }
}

// ------------------------------------------------------------------- tiled
// The product for many rows (prompts), with the tiles going from global memory straight into LDS
// (global_load_lds_dwordx4: a lane's 16 bytes land at base + 16 * lane, no registers, no
// ds_write) and a ring of STAGES k-steps of 32 in LDS, loaded STAGES - 1 steps ahead.
// LDS holds MFMA operands as they are used: a block of 16 rows x 32 k is 1 KB in lane order
// (lane = 16 * (k / 8 % 4) + row % 16), which is the packed weight order, so a packed weight
// block is one contiguous 1 KB load and an operand read is lane * 16 bytes, free of conflicts.
// 16x16x32 MFMA, weight rows first: a lane ends with four consecutive n of one m.
// Workgroup: WNW x WMW waves, each TNB x TMB blocks of 16: BN = 16 TNB WNW, BM = 16 TMB WMW.
template <int N_OUTSTANDING>
__device__ __forceinline__ void wait_vmcnt() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N_OUTSTANDING) : "memory");
}

// The barrier alone: __syncthreads() would first wait for every load in flight, the later stages'
// too, and so undo the ring. What has to have landed is waited for by wait_vmcnt before it; the
// operand reads of the step before are in registers already (the matrix cores have used them).
__device__ __forceinline__ void workgroup_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

template <int EPI, bool PACKED, int TNB, int TMB, int WNW, int WMW, int STAGES, int KS>
__global__ void __launch_bounds__(64 * WNW * WMW)
gemm_dma_kernel(const bf16* __restrict__ X, const bf16* __restrict__ W, void* __restrict__ Cv, int M, int N,
                int K, int ldc, int m_tiles, int n_tiles) {
    constexpr int NW = WNW * WMW;
    constexpr int BN = 16 * TNB * WNW, BM = 16 * TMB * WMW;
    constexpr int WBLK = BN / 16, XBLK = BM / 16, BLKS = WBLK + XBLK;   // 1 KB blocks of a stage
    constexpr int WL = WBLK / NW, XL = XBLK / NW;                      // loads of a wave per stage
    static_assert(WBLK % NW == 0 && XBLK % NW == 0, "blocks must divide over the waves");
    extern __shared__ __attribute__((aligned(1024))) bf16 lds[];        // [STAGES][KS][BLKS][512]

    // Workgroups go round the 8 XCDs, each with an L2 of its own: an XCD takes a run of tiles, and
    // within it bands of 8 tiles in m are walked n first, so that the workgroups that are resident
    // together share both their weight and their activation panels in that L2.
    const int total = m_tiles * n_tiles;
    const int chunk = (total + 7) / 8;
    const int id = (blockIdx.x % 8) * chunk + blockIdx.x / 8;
    if (id >= total) return;
    constexpr int BAND = 8;
    const int band = id / (BAND * n_tiles), in_band = id % (BAND * n_tiles);
    const int band_rows = m_tiles - band * BAND < BAND ? m_tiles - band * BAND : BAND;
    const int n_tile = in_band / band_rows, m_tile = band * BAND + in_band % band_rows;
    const int m0 = m_tile * BM, n0 = n_tile * BN;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // uniform: LDS addresses stay scalar
    const int r16 = lane & 15, g4 = lane >> 4;
    const int wn = wave / WMW, wm = wave % WMW;
    const int k32 = K / 32;              // k-steps of 32 in all
    const int nsteps = k32 / KS;         // stages' worth of them (K is a multiple of 32 KS)

    // this wave's loads: W blocks wave * WL + i, X blocks wave * XL + i
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
    // Stages of 64 k: the activations lie in LDS as rows of 128 bytes, so that a load fetches
    // whole 128-byte lines (8 rows an instruction, 8 lanes a row) instead of half lines twice.
    // The 16-byte chunk c of row r sits at chunk c ^ ((r >> 1) & 7) of its row: the operand reads
    // of 16 rows at one k then fall into 16 different bank groups.
    constexpr bool XROWS = KS == 2;
    constexpr int XR = XROWS ? BM / 8 / NW : 1;                       // row loads of a wave per stage
    static_assert(!XROWS || BM % (8 * NW) == 0, "rows must divide over the waves");
    const bf16* xrsrc[XR];
#pragma unroll
    for (int i = 0; i < XR; ++i) {
        const int r = (wave * XR + i) * 8 + (lane >> 3);
        int m = m0 + r;
        if (m >= M) m = M - 1;
        xrsrc[i] = X + (size_t)m * K + (((lane & 7) ^ ((r >> 1) & 7)) * 8);
    }
    const size_t WSTEP = PACKED ? (size_t)(N / 16) * 512 : 32;

    auto issue = [&](int step, int stage) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            bf16* base = lds + (XROWS ? (size_t)stage * KS * BLKS * 512 + ks * WBLK * 512
                                      : (size_t)(stage * KS + ks) * BLKS * 512);
            const size_t k = (size_t)step * KS + ks;
#pragma unroll
            for (int i = 0; i < WL; ++i)
                __builtin_amdgcn_global_load_lds(
                    (const __attribute__((address_space(1))) void*)(wsrc[i] + k * WSTEP),
                    (__attribute__((address_space(3))) void*)(base + (wave * WL + i) * 512), 16, 0, 0);
            if (!XROWS) {
#pragma unroll
                for (int i = 0; i < XL; ++i)
                    __builtin_amdgcn_global_load_lds(
                        (const __attribute__((address_space(1))) void*)(xsrc[i] + k * 32),
                        (__attribute__((address_space(3))) void*)(base + (WBLK + wave * XL + i) * 512), 16, 0, 0);
            }
        }
        if (XROWS) {
            // the stage's activations follow the weight blocks of its two k-steps: [BM][64]
            bf16* xbase = lds + (size_t)stage * KS * BLKS * 512 + KS * WBLK * 512;
#pragma unroll
            for (int i = 0; i < XR; ++i)
                __builtin_amdgcn_global_load_lds(
                    (const __attribute__((address_space(1))) void*)(xrsrc[i] + (size_t)step * 64),
                    (__attribute__((address_space(3))) void*)(xbase + (wave * XR + i) * 512), 16, 0, 0);
        }
    };

    // 32x32x16 MFMA (it has the higher rate of the two bf16 shapes): an operand is 32 rows x 16 k,
    // lane l = row l % 32, k 8 (l / 32) .. + 8. In the 1 KB blocks of 16 rows x 32 k that is, for the
    // k-half h: block (l % 32) / 16 of a pair of blocks, chunk 16 (2 h + l / 32) + l % 16.
    static_assert(TNB % 2 == 0 && TMB % 2 == 0, "a wave's tile is made of 32 x 32 pieces");
    constexpr int TN32 = TNB / 2, TM32 = TMB / 2;
    const int c32 = lane & 31, g2 = lane >> 5;
    const int lane_off = (c32 >> 4) * 512 + (16 * g2 + (lane & 15)) * 8;   // + 32 * 8 for the second k-half
    f32x16 acc[TN32][TM32];
#pragma unroll
    for (int a = 0; a < TN32; ++a)
#pragma unroll
        for (int b = 0; b < TM32; ++b)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[a][b][i] = 0.f;

    // Operands in two sets of registers: while the matrix cores work on one k-step of 32, the
    // reads of the next one are on their way, so a wave never waits for LDS with nothing to do.
    bf16x8 wv[2][2][TN32], xv[2][2][TM32];       // [set][k-half][piece]
    const int x_swizzle = (c32 >> 1) & 7;           // of this lane's rows: they are c32 + a multiple of 16
    auto read_operands = [&](int set, int stage, int ks) {
        const bf16* base = lds + (XROWS ? (size_t)stage * KS * BLKS * 512 + ks * WBLK * 512
                                        : (size_t)(stage * KS + ks) * BLKS * 512) + lane_off;
        const bf16* xrows = lds + (size_t)stage * KS * BLKS * 512 + KS * WBLK * 512 +
                            ((wm * TMB) * 16 + c32) * 64;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
#pragma unroll
            for (int a = 0; a < TN32; ++a)
                wv[set][h][a] = *(const bf16x8*)(base + (wn * TNB + 2 * a) * 512 + h * 256);
#pragma unroll
            for (int b = 0; b < TM32; ++b) {
                if (XROWS)
                    xv[set][h][b] = *(const bf16x8*)(xrows + b * 32 * 64 + (((4 * ks + 2 * h + g2) ^ x_swizzle) * 8));
                else
                    xv[set][h][b] = *(const bf16x8*)(base + (WBLK + wm * TMB + 2 * b) * 512 + h * 256);
            }
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
        wait_vmcnt<(STAGES - 2) * (XROWS ? WL * KS + XR : (WL + XL) * KS)>();
        workgroup_barrier();
        const int nt = t + STAGES;
        issue(nt < nsteps ? nt : nsteps - 1, nt % STAGES);
    };
    // one step; `first` is the register set that holds its first k-step (a constant once unrolled)
    auto run_step = [&](int first, int t) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const int set = (first + ks) & 1;
            if (ks + 1 < KS) {
                read_operands(set ^ 1, t % STAGES, ks + 1);
            } else if (t + 1 < nsteps) {
                advance(t);
                read_operands(set ^ 1, (t + 1) % STAGES, 0);
            }
            multiply(set);
        }
    };

#pragma unroll
    for (int st = 0; st < STAGES - 1; ++st) issue(st < nsteps ? st : nsteps - 1, st);
    advance(-1);
    read_operands(0, 0, 0);
    if constexpr (KS == 2) {
        // Stages of two k-steps: no branch in the loop (the last step is peeled off), and the work
        // other than MFMAs is dealt out between them by hand: a wave then has an MFMA in the pipe
        // while it issues its reads and loads, also right after the barrier, where the other wave
        // of its SIMD stands at the same place and cannot fill in.
        constexpr int NM = 2 * TN32 * TM32;              // MFMAs of a k-step
        constexpr int NR = 2 * (TN32 + TM32);            // operand reads of a k-step
        constexpr int ND = WL * KS + XR;                 // loads of a stage
        constexpr int SLOTS = NM > 6 ? NM - 4 : NM;      // the last MFMAs cover the latency of the last reads
        auto mfma_one = [&](int set, int j) {
            const int h = j / (TN32 * TM32), a = j / TM32 % TN32, b = j % TM32;
            acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wv[set][h][a], xv[set][h][b], acc[a][b], 0, 0, 0);
        };
        auto read_one = [&](int set, int stage, int ks, int idx) {
            const int h = idx / (TN32 + TM32), r = idx % (TN32 + TM32);
            const bf16* sbase = lds + (size_t)stage * KS * BLKS * 512;
            if (r < TN32) {
                wv[set][h][r] = *(const bf16x8*)(sbase + ks * WBLK * 512 + lane_off + (wn * TNB + 2 * r) * 512 + h * 256);
            } else {
                const int b = r - TN32;
                xv[set][h][b] = *(const bf16x8*)(sbase + KS * WBLK * 512 + ((wm * TMB) * 16 + c32 + b * 32) * 64 +
                                                 (((4 * ks + 2 * h + g2) ^ x_swizzle) * 8));
            }
        };
        auto load_one = [&](int step, int stage, int idx) {
            bf16* sbase = lds + (size_t)stage * KS * BLKS * 512;
            if (idx < WL * KS) {
                const int ks = idx / WL, i = idx % WL;
                __builtin_amdgcn_global_load_lds(
                    (const __attribute__((address_space(1))) void*)(wsrc[i] + ((size_t)step * KS + ks) * WSTEP),
                    (__attribute__((address_space(3))) void*)(sbase + ks * WBLK * 512 + (wave * WL + i) * 512), 16, 0, 0);
            } else {
                const int i = idx - WL * KS;
                __builtin_amdgcn_global_load_lds(
                    (const __attribute__((address_space(1))) void*)(xrsrc[i] + (size_t)step * 64),
                    (__attribute__((address_space(3))) void*)(sbase + KS * WBLK * 512 + (wave * XR + i) * 512), 16, 0, 0);
            }
        };
        for (int t = 0; t + 1 < nsteps; ++t) {
            const int stage = t % STAGES, next_stage = (t + 1) % STAGES;
            // first k-step: its MFMAs, with the reads of the second k-step between them
#pragma unroll
            for (int j = 0; j < NM; ++j) {
                mfma_one(0, j);
#pragma unroll
                for (int o = (j < SLOTS ? j : SLOTS) * NR / SLOTS; o < (j + 1 < SLOTS ? j + 1 : SLOTS) * NR / SLOTS; ++o)
                    read_one(1, stage, 1, o);
                __builtin_amdgcn_sched_barrier(0);
            }
            // second k-step: step t + 1 has landed for everyone and nobody reads this stage any more;
            // between the MFMAs go the loads of step t + STAGES into it, then the reads of step t + 1
            wait_vmcnt<(STAGES - 2) * ND>();
            workgroup_barrier();
            const int nt = t + STAGES < nsteps ? t + STAGES : nsteps - 1;
#pragma unroll
            for (int j = 0; j < NM; ++j) {
                mfma_one(1, j);
#pragma unroll
                for (int o = (j < SLOTS ? j : SLOTS) * (ND + NR) / SLOTS;
                     o < (j + 1 < SLOTS ? j + 1 : SLOTS) * (ND + NR) / SLOTS; ++o) {
                    if (o < ND) load_one(nt, stage, o);
                    else read_one(0, next_stage, 0, o - ND);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        {
            const int stage = (nsteps - 1) % STAGES;
#pragma unroll
            for (int j = 0; j < NM; ++j) {
                mfma_one(0, j);
#pragma unroll
                for (int o = (j < SLOTS ? j : SLOTS) * NR / SLOTS; o < (j + 1 < SLOTS ? j + 1 : SLOTS) * NR / SLOTS; ++o)
                    read_one(1, stage, 1, o);
                __builtin_amdgcn_sched_barrier(0);
            }
            multiply(1);
        }
    } else if (KS % 2 == 0) {
        for (int t = 0; t < nsteps; ++t) run_step(0, t);
    } else {
        for (int t = 0; t < nsteps; t += 2) {
            run_step(0, t);
            if (t + 1 < nsteps) run_step(1, t + 1);
        }
    }
    wait_vmcnt<0>();      // the loads past the end (repeats of the last step) have landed too

    // lane: m = m0 + (wm * TMB + 2 b) * 16 + c32 ; register 4 q + j of a piece:
    // n = n0 + (wn * TNB + 2 a) * 16 + 8 q + 4 g2 + j, four consecutive n for each q
#pragma unroll
    for (int b = 0; b < TM32; ++b) {
        const int m = m0 + (wm * TMB + 2 * b) * 16 + c32;
        if (m >= M) continue;
        if (EPI == EPI_SWIGLU) {
            bf16* C = (bf16*)Cv;
#pragma unroll
            for (int a = 0; a < TN32; ++a)
#pragma unroll
                for (int q = 0; q < 2; ++q) {
                    // rows 0..15 of the piece are gate rows, 16..31 the up rows of the same outputs
                    const int n = (n0 + (wn * TNB + 2 * a) * 16) / 2 + 8 * q + 4 * g2;
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
                    const int n = n0 + (wn * TNB + 2 * a) * 16 + 8 * q + 4 * g2;
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

template <int TNB, int TMB, int WNW, int WMW, int STAGES, int KS>
static int launch_dma(const void* X, const void* W, void* C, int M, int N, int K, int ldc, int epi, int packed,
                      hipStream_t stream) {
    constexpr int BN = 16 * TNB * WNW, BM = 16 * TMB * WMW;
    const int m_tiles = (M + BM - 1) / BM, n_tiles = (N + BN - 1) / BN;
    const long total = (long)m_tiles * n_tiles;
    HB_REQUIRE(total < (1l << 30), "gemm_mfma: too many tiles");
    const int blocks = (int)((total + 7) / 8 * 8);
    HB_REQUIRE(K % (32 * KS) == 0, "gemm_mfma: K=%d is no multiple of %d", K, 32 * KS);
    const size_t lds = (size_t)STAGES * KS * (BN + BM) / 16 * 1024;
    const bf16* x = (const bf16*)X;
    const bf16* w = (const bf16*)W;
#define DMA_GO(EPIV, PK)                                                                            \
    do {                                                                                            \
        auto kern = gemm_dma_kernel<EPIV, PK, TNB, TMB, WNW, WMW, STAGES, KS>;                          \
        if (lds > 64 * 1024) {                                                                      \
            static bool raised = false;                                                             \
            if (!raised) {                                                                          \
                hipError_t e = hipFuncSetAttribute((const void*)kern,                               \
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds); \
                HB_REQUIRE(e == hipSuccess, "gemm_mfma: cannot have %zu bytes of LDS: %s", lds,     \
                           hipGetErrorString(e));                                                   \
                raised = true;                                                                      \
            }                                                                                       \
        }                                                                                           \
        kern<<<blocks, 64 * WNW * WMW, lds, stream>>>(x, w, C, M, N, K, ldc, m_tiles, n_tiles);     \
    } while (0)
    if (packed) {
        if (epi == EPI_STORE) DMA_GO(EPI_STORE, true);
        else if (epi == EPI_ADD) DMA_GO(EPI_ADD, true);
        else DMA_GO(EPI_SWIGLU, true);
    } else {
        if (epi == EPI_STORE) DMA_GO(EPI_STORE, false);
        else if (epi == EPI_ADD) DMA_GO(EPI_ADD, false);
        else DMA_GO(EPI_SWIGLU, false);
    }
#undef DMA_GO
    HB_CHECK_LAUNCH("gemm_dma");
    return 0;
}

// C (+)= X @ W^T. X [M, K] bf16, W [N, K] bf16. epi 0: C f32 [M, N] stored; 1: added to;
// 2: W's rows are gate/up interleaved in blocks of 16 and C is bf16 [M, N / 2] = silu(gate) * up.
// packed != 0: W is stored as [K / 32][N / 16][64 lanes][8]: lane = 16 * (k / 8 % 4) + n % 16.
// All blocks of one k-step lie together: workgroups that advance through K side by side read one
// contiguous stretch of memory at a time, as a streaming copy would.
// workspace: float scratch for K cut into slices (17 to 64 rows); without it K is not cut.
// norm_w != null: X is the float32 residual stream [M, K] and the product is RMSNorm(X; norm_w, eps) W^T
// (M <= 64 only, never with the add epilogue).
extern "C" int hb_gemm_mfma(const void* X, const void* W, void* C, int M, int N, int K, int ldc, int epi,
                            int packed, const float* norm_w, float eps, int tile_hint, float* workspace,
                            size_t workspace_floats, hipStream_t stream) {
    HB_REQUIRE(!norm_w || (M <= 16 && epi != EPI_ADD && (epi == EPI_SWIGLU || N >= 16384)),
               "gemm_mfma: the fused norm takes M <= 16, N >= 16384 and no add");
    HB_REQUIRE(!packed || N % 16 == 0, "gemm_mfma: packed weights need N %% 16 == 0");
    HB_REQUIRE(M > 0 && N > 0 && K > 0, "gemm_mfma: empty problem (M=%d, N=%d, K=%d)", M, N, K);
    HB_REQUIRE(epi >= 0 && epi <= 2, "gemm_mfma: unknown epilogue %d", epi);
    HB_REQUIRE(K % 32 == 0, "gemm_mfma: K=%d is no multiple of 32", K);
    HB_REQUIRE(epi != EPI_SWIGLU || N % 32 == 0, "gemm_mfma: the SwiGLU epilogue needs N %% 32 == 0");
    HB_REQUIRE(ldc >= (epi == EPI_SWIGLU ? N / 2 : N), "gemm_mfma: output row stride %d too small", ldc);
    if (M <= 64) {
        if (M <= 16) pick_skinny<1>(X, W, C, M, N, K, ldc, epi, packed, norm_w, eps, stream, workspace, workspace_floats);
        else if (M <= 32) pick_skinny<2>(X, W, C, M, N, K, ldc, epi, packed, norm_w, eps, stream, workspace, workspace_floats);
        else if (M <= 48) pick_skinny<3>(X, W, C, M, N, K, ldc, epi, packed, norm_w, eps, stream, workspace, workspace_floats);
        else pick_skinny<4>(X, W, C, M, N, K, ldc, epi, packed, norm_w, eps, stream, workspace, workspace_floats);
        HB_CHECK_LAUNCH("gemm_skinny");
        return 0;
    }
    // tile_hint: 0 = choose (otherwise a variant by number, for measurements and tests).
    // 256 x 256 tiles do the most arithmetic per byte moved, but one fits a CU at a time: they pay
    // when there are enough of them for most of the 256 CUs; otherwise 128 x 128, two to a CU.
    int tile = tile_hint;
    if (tile == 0) {
        const long big = (long)((M + 255) / 256) * ((N + 255) / 256);
        tile = K % 64 ? 123 : (big >= 192 ? 185 : 122);
    }
    switch (tile) {
        case 185: return launch_dma<8, 4, 2, 4, 2, 2>(X, W, C, M, N, K, ldc, epi, packed, stream);   // 256 x 256, 2 stages of 64 k
        case 122: return launch_dma<4, 4, 2, 2, 2, 2>(X, W, C, M, N, K, ldc, epi, packed, stream);   // 128 x 128, 2 stages of 64 k
        case 123: return launch_dma<4, 4, 2, 2, 4, 1>(X, W, C, M, N, K, ldc, epi, packed, stream);   // 128 x 128, 4 stages of 32 k
        case 188: return launch_dma<8, 8, 2, 2, 2, 2>(X, W, C, M, N, K, ldc, epi, packed, stream);   // 256 x 256, 4 waves
        default: HB_REQUIRE(false, "gemm_mfma: unknown tile %d", tile);
    }
    return 0;
}
