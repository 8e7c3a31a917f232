// Row-wise kernels of the decoder: embedding gather, RMSNorm, the fused
// per-head norm + rotation + cache write, and SwiGLU. All arithmetic is float32;
// the template parameters are the storage types of inputs and outputs.
// What each computes, in xigh/herbert-rs:
//   embedding        crates/backends/backend_common/src/generic_model.rs:104-111 (no multiplier; an id >= V is an error);
//                    crates/backends/backend_vulkan/shaders/embedding.comp:20-27
//   RMSNorm          crates/backends/backend_common/src/kernels.rs:54-64: x * 1 / sqrt(sum(x^2) / dim + eps) * w, eps inside
//                    the root, plain weight; crates/backends/backend_vulkan/shaders/rms_norm_batch.comp:25-41
//   per-head norm    crates/backends/backend_common/src/generic_attention/mod.rs:62-76 (before the rotation, the same eps,
//                    one weight [hd] for all heads, values untouched); backend_vulkan/shaders/head_rms_norm.comp:24-41
//   rotation         crates/backends/backend_common/src/kernels.rs:739-759 (pairs (j, j + R/2): x0 c - x1 s, x0 s + x1 c;
//                    elements from R on unchanged); tables crates/backends/backend_common/src/loader_common.rs:179-202
//   the three fused  crates/backends/backend_metal/shaders/head_norm_rope_kv_append.metal:37-110 (norm, rotation, append)
//   SwiGLU           crates/backends/backend_common/src/kernels.rs:676-687: g / (1 + exp(-g)) * u
#include "common.h"

HB_MODULE_ERROR_SLOT()

// ---------------------------------------------------------------- embedding
// x[t, :] = float(table[ids[t], :]); the residual stream is float32.
// PACKED: the table is stored in the MFMA kernels' order [H / 32][V / 16][64 lanes][8], element
// (n, k) at ((k / 32 * (V / 16) + n / 16) * 64 + (k / 8 % 4) * 16 + n % 16) * 8 + k % 8.
template <class TW, bool PACKED>
__global__ void embed_kernel(const int* __restrict__ ids, const TW* __restrict__ table,
                             float* __restrict__ x, int H, int V) {
    const int t = blockIdx.x;
    const int n = ids[t];
    float* out = x + (size_t)t * H;
    if ((unsigned)n >= (unsigned)V) {
        // The host checks the ids it sees; ids that come from the GPU (a sampler's output fed to the
        // next step) cannot be: a bad one reads nothing and makes its row NaN, which shows.
        for (int i = threadIdx.x; i < H; i += blockDim.x) out[i] = __uint_as_float(0x7fc00000u);
        return;
    }
    if (PACKED) {
        const TW* blk = table + (size_t)(n / 16) * 512 + (n % 16) * 8;
        const size_t plane = (size_t)(V / 16) * 512;
        for (int k = threadIdx.x; k < H; k += blockDim.x)
            out[k] = hb_to_float(blk[(size_t)(k / 32) * plane + ((k / 8) % 4) * 128 + (k % 8)]);
    } else {
        const TW* row = table + (size_t)n * H;
        if (sizeof(TW) == 2 && H % 8 == 0) {
            // eight bfloat16 a load (rows of a table whose width is a multiple of 8 start at 16 bytes)
            for (int i = threadIdx.x * 8; i < H; i += blockDim.x * 8) {
                const uint4 raw = *(const uint4*)(row + i);
                const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
                float v[8];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    v[2 * e] = __uint_as_float(w[e] << 16);
                    v[2 * e + 1] = __uint_as_float(w[e] & 0xffff0000u);
                }
                *(float4*)(out + i) = float4{v[0], v[1], v[2], v[3]};
                *(float4*)(out + i + 4) = float4{v[4], v[5], v[6], v[7]};
            }
            return;
        }
        for (int i = threadIdx.x; i < H; i += blockDim.x) out[i] = hb_to_float(row[i]);
    }
}

extern "C" int hb_embed(const int* ids, const void* table, int table_dtype, float* x, int T, int H, int V,
                        int packed, hipStream_t stream) {
    HB_REQUIRE(T > 0 && H > 0, "embed: empty input (T=%d, H=%d)", T, H);
    HB_REQUIRE(!packed || (table_dtype == HB_BF16 && H % 32 == 0 && V % 16 == 0),
               "embed: a packed table is bfloat16 with a width in steps of 32 and rows in steps of 16");
    if (table_dtype == HB_F32)
        embed_kernel<float, false><<<T, 256, 0, stream>>>(ids, (const float*)table, x, H, V);
    else if (table_dtype == HB_BF16 && packed)
        embed_kernel<bf16, true><<<T, 256, 0, stream>>>(ids, (const bf16*)table, x, H, V);
    else if (table_dtype == HB_BF16)
        embed_kernel<bf16, false><<<T, 256, 0, stream>>>(ids, (const bf16*)table, x, H, V);
    else
        HB_REQUIRE(false, "embed: unknown table dtype %d", table_dtype);
    HB_CHECK_LAUNCH("embed");
    return 0;
}

// ------------------------------------------------------------------ RMSNorm
// y[r, :] = x[src(r), :] * rsqrt(mean(x^2) + eps) * w ; src(r) = rows ? rows[r] : r.
// One block per output row; the sum's order depends on H and the block size only.
template <class TOut>
__global__ void rmsnorm_kernel(const float* __restrict__ x, const float* __restrict__ w,
                               TOut* __restrict__ y, const int* __restrict__ rows, int H, float eps) {
    __shared__ float red[16];
    const int r = blockIdx.x;
    const float* in = x + (size_t)(rows ? rows[r] : r) * H;
    TOut* out = y + (size_t)r * H;
    float ss = 0.f;
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
        const float v = in[i];
        ss += v * v;
    }
    ss = hb_block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)H + eps);
    for (int i = threadIdx.x; i < H; i += blockDim.x) out[i] = hb_from_float<TOut>(in[i] * inv * w[i]);
}

// The same for rows that fit the registers of one block (H in steps of 4, at most 8192): every
// element is loaded once, 16 bytes a lane, all loads in flight together.
typedef float hb_f4 __attribute__((ext_vector_type(4)));
// four neighbours of a row in one store (rows start at multiples of four elements)
__device__ __forceinline__ void store_four(float* out, hb_f4 v) { *(hb_f4*)out = v; }
__device__ __forceinline__ void store_four(bf16* out, hb_f4 v) {
    // (two conversions a register, round to nearest even as hb_from_float)
    typedef __bf16 hb_b2 __attribute__((ext_vector_type(2)));
    const hb_b2 lo = {(__bf16)v[0], (__bf16)v[1]}, hi = {(__bf16)v[2], (__bf16)v[3]};
    *(uint2*)out = uint2{__builtin_bit_cast(uint32_t, lo), __builtin_bit_cast(uint32_t, hi)};
}
template <class TOut>
__global__ void __launch_bounds__(256)
rmsnorm_row_kernel(const float* __restrict__ x, const float* __restrict__ w, TOut* __restrict__ y,
                   const int* __restrict__ rows, int H, float eps) {
    __shared__ float red[16];
    const int r = blockIdx.x;
    const hb_f4* in = (const hb_f4*)(x + (size_t)(rows ? rows[r] : r) * H);
    const hb_f4* w4 = (const hb_f4*)w;
    const int nv = H / 4;
    hb_f4 v[8], g[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) {
        const int i = threadIdx.x + 256 * c;
        if (i < nv) {
            v[c] = in[i];
            g[c] = w4[i];
        } else {
            v[c] = g[c] = hb_f4{0.f, 0.f, 0.f, 0.f};
        }
    }
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < 8; ++c) ss += v[c][0] * v[c][0] + v[c][1] * v[c][1] + v[c][2] * v[c][2] + v[c][3] * v[c][3];
    ss = hb_block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)H + eps);
    TOut* out = y + (size_t)r * H;
#pragma unroll
    for (int c = 0; c < 8; ++c) {
        const int i = threadIdx.x + 256 * c;
        if (i < nv) {
            // (element by element: written as a product of vectors this took 380 registers)
            hb_f4 r;
#pragma unroll
            for (int e = 0; e < 4; ++e) r[e] = v[c][e] * inv * g[c][e];
            store_four(out + 4 * i, r);
        }
    }
}

extern "C" int hb_rmsnorm(const float* x, const float* w, void* y, int y_dtype, const int* rows, int R,
                          int H, float eps, hipStream_t stream) {
    HB_REQUIRE(R > 0 && H > 0, "rmsnorm: empty input (R=%d, H=%d)", R, H);
    HB_REQUIRE(y_dtype == HB_F32 || y_dtype == HB_BF16, "rmsnorm: unknown output dtype %d", y_dtype);
    if (H % 4 == 0 && H >= 1024 && H <= 8192) {
        if (y_dtype == HB_F32)
            rmsnorm_row_kernel<float><<<R, 256, 0, stream>>>(x, w, (float*)y, rows, H, eps);
        else
            rmsnorm_row_kernel<bf16><<<R, 256, 0, stream>>>(x, w, (bf16*)y, rows, H, eps);
    } else {
        const int threads = H >= 1024 ? 256 : 64;
        if (y_dtype == HB_F32)
            rmsnorm_kernel<float><<<R, threads, 0, stream>>>(x, w, (float*)y, rows, H, eps);
        else
            rmsnorm_kernel<bf16><<<R, threads, 0, stream>>>(x, w, (bf16*)y, rows, H, eps);
    }
    HB_CHECK_LAUNCH("rmsnorm");
    return 0;
}

// ------------------------------------- per-head norm + rotation + cache write
// One wave per (token, head) of the fused projection row [q heads | k heads | v heads].
//   q heads: optional RMSNorm over the head, optional rotation, written to q_out.
//   k heads: the same, written to the key pages of the token's slot.
//   v heads: copied to the value pages, which are transposed: [page, kv head, hd, token].
// Rotation pairs dim j with j + R/2 (R = rot_dims), angle table [max_pos, R/2].
// The page of position p of a slot is page_table[slot * max_pages + p / page_size].
#define HB_MAX_HEAD_DIM 512

template <class TQ, class TC>
__global__ void qk_norm_rope_write_kernel(
    const float* __restrict__ qkv, int ld_qkv, const float* __restrict__ q_norm_w,
    const float* __restrict__ k_norm_w, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    int rot_dims, const int* __restrict__ positions, const int* __restrict__ seq_of,
    const int* __restrict__ slots, const int* __restrict__ page_table, int max_pages, int page_size,
    TQ* __restrict__ q_out, TC* __restrict__ k_cache, TC* __restrict__ v_cache, int nq, int nkv, int hd,
    float eps) {
    __shared__ float vec[HB_MAX_HEAD_DIM];
    const int t = blockIdx.x;
    const int h = blockIdx.y;
    const int lane = threadIdx.x;
    const float* src = qkv + (size_t)t * ld_qkv + (size_t)h * hd;
    const bool is_q = h < nq;
    const bool is_v = h >= nq + nkv;
    const int pos = positions[t];

    float ss = 0.f;
    for (int d = lane; d < hd; d += HB_WAVE) {
        const float v = src[d];
        vec[d] = v;
        ss += v * v;
    }
    ss = hb_wave_sum(ss);
    __syncthreads();

    const float* norm_w = is_q ? q_norm_w : k_norm_w;
    const bool do_norm = !is_v && norm_w != nullptr;
    const bool do_rope = !is_v && cos_t != nullptr;
    const float inv = do_norm ? 1.0f / sqrtf(ss / (float)hd + eps) : 1.0f;
    const int half = rot_dims / 2;

    size_t dst_base = 0;      // keys: start of the token's row; values: start of the (page, head) block
    if (!is_q) {
        const int slot = slots[seq_of[t]];
        const int page = page_table[(size_t)slot * max_pages + pos / page_size];
        const int kvh = is_v ? h - nq - nkv : h - nq;
        dst_base = ((size_t)page * nkv + kvh) * page_size * hd;
        if (!is_v) dst_base += (size_t)(pos % page_size) * hd;
    }
    const int in_page = pos % page_size;

    for (int d = lane; d < hd; d += HB_WAVE) {
        float out;
        if (do_rope && d < rot_dims) {
            const int j = d < half ? d : d - half;
            const float c = cos_t[(size_t)pos * half + j];
            const float s = sin_t[(size_t)pos * half + j];
            float x0 = vec[j], x1 = vec[j + half];
            if (do_norm) {
                x0 = x0 * inv * norm_w[j];
                x1 = x1 * inv * norm_w[j + half];
            }
            out = d < half ? x0 * c - x1 * s : x0 * s + x1 * c;
        } else {
            out = vec[d];
            if (do_norm) out = out * inv * norm_w[d];
        }
        if (is_q)
            q_out[(size_t)t * nq * hd + (size_t)h * hd + d] = hb_from_float<TQ>(out);
        else if (is_v)
            v_cache[dst_base + (size_t)d * page_size + in_page] = hb_from_float<TC>(out);
        else
            k_cache[dst_base + d] = hb_from_float<TC>(out);
    }
}

// The same for many tokens (prompts), bfloat16 output, rotation over the whole head or none,
// head size in steps of 8 up to 128, rows of the projection 16-byte aligned: a workgroup takes 64
// consecutive tokens of one head. Query and key heads: half a wave a token, 16 bytes a lane.
// Value heads go through LDS, so that the transposed pages are written along the tokens: lane =
// token, 64 consecutive tokens of a page are one 128-byte line.
// QS > 1: the projection was cut into QS slices of K whose sums lie slice_stride floats apart
// behind qkv; they are added up in their order as they are loaded.
#define HB_TILED_HEAD_DIM 128
template <class TQ, class TC, int QS>
__global__ void __launch_bounds__(256) qk_norm_rope_write_tiled_kernel(
    const float* __restrict__ qkv, int ld_qkv, size_t slice_stride, const float* __restrict__ q_norm_w,
    const float* __restrict__ k_norm_w, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    const int* __restrict__ positions, const int* __restrict__ seq_of, const int* __restrict__ slots,
    const int* __restrict__ page_table, int max_pages, int page_size, TQ* __restrict__ q_out,
    TC* __restrict__ k_cache, TC* __restrict__ v_cache, int T, int nq, int nkv, int hd, float eps) {
    __shared__ float vt[64][HB_TILED_HEAD_DIM + 1];
    const int t0 = blockIdx.x * 64, h = blockIdx.y;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const bool is_q = h < nq, is_v = h >= nq + nkv;
    const int half = hd / 2;
    auto summed4 = [&](const float* p) {
        hb_f4 part[QS];
#pragma unroll
        for (int i = 0; i < QS; ++i) part[i] = *(const hb_f4*)(p + (size_t)i * slice_stride);
        hb_f4 sum = part[0];
#pragma unroll
        for (int i = 1; i < QS; ++i) sum += part[i];
        return sum;
    };
    if (is_v) {
        const int kvh = h - nq - nkv;
        const int q4 = hd / 4;                       // 16-byte chunks of a row
        for (int idx = tid; idx < 64 * q4; idx += 256) {
            const int r = idx / q4, c = (idx - r * q4) * 4;
            const int t = t0 + r;
            hb_f4 v = {0.f, 0.f, 0.f, 0.f};
            if (t < T) v = summed4(qkv + (size_t)t * ld_qkv + (size_t)h * hd + c);
#pragma unroll
            for (int e = 0; e < 4; ++e) vt[r][c + e] = v[e];
        }
        __syncthreads();
        const int t = t0 + lane;
        if (t >= T) return;
        const int pos = positions[t];
        const int page = page_table[(size_t)slots[seq_of[t]] * max_pages + pos / page_size];
        TC* dst = v_cache + ((size_t)page * nkv + kvh) * page_size * hd + pos % page_size;
        for (int d = wave; d < hd; d += 4) dst[(size_t)d * page_size] = hb_from_float<TC>(vt[lane][d]);
        return;
    }
    // Query and key heads: half a wave a token, a lane four consecutive elements (16 bytes in, 8
    // out); the lanes l < hd / 8 hold the first half of the head, their partners l + hd / 8 the
    // elements they are rotated with. A wave's 16 tokens go in two rounds of 8 (4 passes of 2
    // tokens): all loads of a round go out before anything waits for them.
    const float* norm_w = is_q ? q_norm_w : k_norm_w;
    const int l = lane & 31, sub = lane >> 5;
    const int eighth = hd / 8;
    const bool mine = l < 2 * eighth;
    const bool first = l < eighth;
    const int d0 = mine ? 4 * l : 0;
    const int j0 = mine && !first ? d0 - half : d0;              // where this lane's angles lie
    const int partner = (lane & 32) + (mine ? (first ? l + eighth : l - eighth) : l);
    hb_f4 w = {1.f, 1.f, 1.f, 1.f};
    if (norm_w && mine) w = *(const hb_f4*)(norm_w + d0);
#pragma unroll
    for (int round = 0; round < 2; ++round) {
        hb_f4 x[4], c[4], sn[4];
        int pos[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int t = t0 + 16 * wave + 8 * round + 2 * u + sub;
            const int tc = t < T ? t : T - 1;
            pos[u] = positions[tc];
            x[u] = hb_f4{0.f, 0.f, 0.f, 0.f};
            if (mine) x[u] = summed4(qkv + (size_t)tc * ld_qkv + (size_t)h * hd + d0);
        }
        if (cos_t) {
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                c[u] = *(const hb_f4*)(cos_t + (size_t)pos[u] * half + j0);
                sn[u] = *(const hb_f4*)(sin_t + (size_t)pos[u] * half + j0);
            }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int t = t0 + 16 * wave + 8 * round + 2 * u + sub;
            hb_f4 a = x[u];
            if (norm_w) {
                float ss = a[0] * a[0] + a[1] * a[1] + a[2] * a[2] + a[3] * a[3];
#pragma unroll
                for (int d = 1; d < 32; d <<= 1) ss += __shfl_xor(ss, d, 64);
                const float inv = 1.0f / sqrtf(ss / (float)hd + eps);
#pragma unroll
                for (int e = 0; e < 4; ++e) a[e] = a[e] * inv * w[e];
            }
            if (cos_t) {
                hb_f4 o;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float other = __shfl(a[e], partner, 64);
                    // first half: x0 c - x1 s; second half: x0 s + x1 c (x0 the partner's element)
                    o[e] = first ? a[e] * c[u][e] - other * sn[u][e] : other * sn[u][e] + a[e] * c[u][e];
                }
                a = o;
            }
            if (!mine || t >= T) continue;
            TQ packed[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) packed[e] = hb_from_float<TQ>(a[e]);
            if (is_q) {
                *(uint2*)(q_out + ((size_t)t * nq + h) * hd + d0) = *(const uint2*)packed;
            } else {
                const int page = page_table[(size_t)slots[seq_of[t]] * max_pages + pos[u] / page_size];
                *(uint2*)(k_cache + (((size_t)page * nkv + (h - nq)) * page_size + pos[u] % page_size) * hd + d0) =
                    *(const uint2*)packed;
            }
        }
    }
}

extern "C" int hb_qk_norm_rope_write(const float* qkv, int ld_qkv, const float* q_norm_w,
                                     const float* k_norm_w, const float* cos_t, const float* sin_t,
                                     int rot_dims, const int* positions, const int* seq_of,
                                     const int* slots, const int* page_table, int max_pages,
                                     int page_size, void* q_out, void* k_cache, void* v_cache, int dtype,
                                     int T, int nq, int nkv, int hd, float eps, int write_kv,
                                     int qkv_slices, size_t slice_stride, hipStream_t stream) {
    HB_REQUIRE(T > 0 && nq > 0 && nkv > 0, "qk_norm_rope_write: empty input");
    HB_REQUIRE(hd > 0 && hd <= HB_MAX_HEAD_DIM, "qk_norm_rope_write: head_dim %d not in 1..%d", hd,
               HB_MAX_HEAD_DIM);
    HB_REQUIRE(rot_dims % 2 == 0 && rot_dims >= 0 && rot_dims <= hd,
               "qk_norm_rope_write: rotary dims %d must be even and <= head_dim %d", rot_dims, hd);
    // write_kv == 0: the row holds query heads only and the cache is left alone
    const int heads = nq + (write_kv ? 2 * nkv : 0);
    HB_REQUIRE(ld_qkv >= heads * hd, "qk_norm_rope_write: row stride %d too small", ld_qkv);
    HB_REQUIRE(heads <= 65535, "qk_norm_rope_write: too many heads for the grid");
    if (dtype == HB_BF16 && write_kv && T >= 64 && hd <= HB_TILED_HEAD_DIM && hd % 8 == 0 && ld_qkv % 4 == 0 &&
        slice_stride % 4 == 0 && ((uintptr_t)qkv & 15) == 0 &&
        (cos_t == nullptr || rot_dims == hd) && (T + 63) / 64 <= 0x7fffffff) {
        dim3 tiles((T + 63) / 64, heads);
        HB_REQUIRE(qkv_slices == 1 || slice_stride >= (size_t)T * ld_qkv, "qk_norm_rope_write: slices overlap");
#define TILED_GO(QSV)                                                                                          \
    qk_norm_rope_write_tiled_kernel<bf16, bf16, QSV><<<tiles, 256, 0, stream>>>(                              \
        qkv, ld_qkv, slice_stride, q_norm_w, k_norm_w, cos_t, sin_t, positions, seq_of, slots, page_table,    \
        max_pages, page_size, (bf16*)q_out, (bf16*)k_cache, (bf16*)v_cache, T, nq, nkv, hd, eps)
        if (qkv_slices == 1) TILED_GO(1);
        else if (qkv_slices == 2) TILED_GO(2);
        else if (qkv_slices == 4) TILED_GO(4);
        else if (qkv_slices == 8) TILED_GO(8);
        else HB_REQUIRE(false, "qk_norm_rope_write: %d slices of the projection are not taken", qkv_slices);
#undef TILED_GO
        HB_CHECK_LAUNCH("qk_norm_rope_write_tiled");
        return 0;
    }
    HB_REQUIRE(qkv_slices == 1, "qk_norm_rope_write: only the kernel for bfloat16 prompts of 64 tokens or more adds up slices");
    dim3 grid(T, heads);
    if (dtype == HB_F32)
        qk_norm_rope_write_kernel<float, float><<<grid, HB_WAVE, 0, stream>>>(
            qkv, ld_qkv, q_norm_w, k_norm_w, cos_t, sin_t, rot_dims, positions, seq_of, slots,
            page_table, max_pages, page_size, (float*)q_out, (float*)k_cache, (float*)v_cache, nq, nkv,
            hd, eps);
    else if (dtype == HB_BF16)
        qk_norm_rope_write_kernel<bf16, bf16><<<grid, HB_WAVE, 0, stream>>>(
            qkv, ld_qkv, q_norm_w, k_norm_w, cos_t, sin_t, rot_dims, positions, seq_of, slots,
            page_table, max_pages, page_size, (bf16*)q_out, (bf16*)k_cache, (bf16*)v_cache, nq, nkv, hd,
            eps);
    else
        HB_REQUIRE(false, "qk_norm_rope_write: unknown dtype %d", dtype);
    HB_CHECK_LAUNCH("qk_norm_rope_write");
    return 0;
}

// ------------------------------------------------------------------- SwiGLU
// act[t, i] = silu(gu[t, i]) * gu[t, I + i], silu(g) = g / (1 + exp(-g)).
template <class TOut>
__global__ void swiglu_kernel(const float* __restrict__ gu, TOut* __restrict__ act, int I, size_t total) {
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const size_t t = idx / I;
    const int i = (int)(idx - t * I);
    const float g = gu[t * 2 * I + i];
    const float u = gu[t * 2 * I + I + i];
    act[idx] = hb_from_float<TOut>(g / (1.0f + expf(-g)) * u);
}

extern "C" int hb_swiglu(const float* gu, void* act, int act_dtype, int T, int I, hipStream_t stream) {
    HB_REQUIRE(T > 0 && I > 0, "swiglu: empty input");
    const size_t total = (size_t)T * I;
    const unsigned blocks = (unsigned)((total + 255) / 256);
    if (act_dtype == HB_F32)
        swiglu_kernel<float><<<blocks, 256, 0, stream>>>(gu, (float*)act, I, total);
    else if (act_dtype == HB_BF16)
        swiglu_kernel<bf16><<<blocks, 256, 0, stream>>>(gu, (bf16*)act, I, total);
    else
        HB_REQUIRE(false, "swiglu: unknown output dtype %d", act_dtype);
    HB_CHECK_LAUNCH("swiglu");
    return 0;
}

// ------------------------------------------------------------------ fill
// A small fill kernel: clears memory inside captured graphs, where a memset node may not stand.
__global__ void fill_u32_kernel(uint32_t* p, uint32_t v, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

extern "C" int hb_fill_u32(void* p, uint32_t value, size_t n, hipStream_t stream) {
    if (n == 0) return 0;
    fill_u32_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>((uint32_t*)p, value, n);
    HB_CHECK_LAUNCH("fill_u32");
    return 0;
}
