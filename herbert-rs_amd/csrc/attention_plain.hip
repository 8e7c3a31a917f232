// Plain attention over the paged cache, float32 arithmetic, any storage types,
// any head size up to 512, any number of heads and groups.
// One wave per (token, query head). The keys a query at position p sees are
// [max(0, p + 1 - window), p] (window 0 = all keys from 0). They are walked in
// chunks of 64 that start at multiples of 64 of the absolute position, with an
// online softmax: the chunking, and so the rounding, depends on the positions only,
// not on how the tokens were cut into steps or batches.
// In xigh/herbert-rs: scores q . k / sqrt(hd), query head h on kv head h / (nq / nkv)
// (crates/backends/backend_common/src/generic_attention/decode.rs:126), causal by count
// (crates/backends/backend_common/src/generic_attention/prefill/kernel_f32.rs:65-67), online softmax and
// sum of p v (kernel_f32.rs:83-110; decoding: crates/backends/backend_common/src/attention_common.rs:141-178),
// all float32. The window is not in the reference, which never reads those keys.
#include "common.h"
#include <math.h>

HB_MODULE_ERROR_SLOT()

#define HB_MAX_HEAD_DIM 512
#define ACC_REGS (HB_MAX_HEAD_DIM / HB_WAVE)

template <class TQ, class TC, class TO>
__global__ void __launch_bounds__(HB_WAVE)
attention_plain_kernel(const TQ* __restrict__ q, const TC* __restrict__ k_cache,
                       const TC* __restrict__ v_cache, TO* __restrict__ out,
                       const int* __restrict__ positions, const int* __restrict__ seq_of,
                       const int* __restrict__ slots, const int* __restrict__ page_table, int max_pages,
                       int page_size, int nq, int nkv, int hd, float scale, int window) {
    __shared__ float qs[HB_MAX_HEAD_DIM];
    __shared__ float ps[HB_WAVE];
    const int t = blockIdx.x;
    const int h = blockIdx.y;
    const int lane = threadIdx.x;
    const int g = h / (nq / nkv);
    const int pos = positions[t];
    const int slot = slots[seq_of[t]];
    const int* pt = page_table + (size_t)slot * max_pages;

    const TQ* qrow = q + ((size_t)t * nq + h) * hd;
    for (int d = lane; d < hd; d += HB_WAVE) qs[d] = hb_to_float(qrow[d]);
    __syncthreads();

    const int hi = pos + 1;
    const int lo = (window > 0 && hi > window) ? hi - window : 0;
    float m = -INFINITY, l = 0.f;
    float acc[ACC_REGS];
#pragma unroll
    for (int i = 0; i < ACC_REGS; ++i) acc[i] = 0.f;

    for (int c = (lo / HB_WAVE) * HB_WAVE; c < hi; c += HB_WAVE) {
        const int j = c + lane;
        const bool valid = j >= lo && j < hi;
        float s = -INFINITY;
        if (valid) {
            const int page = pt[j / page_size];
            const TC* kr = k_cache + (((size_t)page * nkv + g) * page_size + (j % page_size)) * hd;
            float dot = 0.f;
            for (int d = 0; d < hd; ++d) dot = fmaf(qs[d], hb_to_float(kr[d]), dot);
            s = dot * scale;
        }
        const float m_new = fmaxf(m, hb_wave_max(s));
        const float corr = expf(m - m_new);
        const float p = valid ? expf(s - m_new) : 0.f;
        l = l * corr + hb_wave_sum(p);
        m = m_new;
        __syncthreads();
        ps[lane] = p;
        __syncthreads();
        const int jj0 = lo > c ? lo - c : 0;
        const int jj1 = hi - c < HB_WAVE ? hi - c : HB_WAVE;
#pragma unroll
        for (int i = 0; i < ACC_REGS; ++i) acc[i] *= corr;
        for (int jj = jj0; jj < jj1; ++jj) {
            const int jv = c + jj;
            const int page = pt[jv / page_size];
            // values are stored transposed: [page, kv head, hd, token]
            const TC* vr = v_cache + ((size_t)page * nkv + g) * page_size * hd + (jv % page_size);
            const float pj = ps[jj];
#pragma unroll
            for (int i = 0; i < ACC_REGS; ++i) {
                const int d = lane + HB_WAVE * i;
                if (d < hd) acc[i] = fmaf(pj, hb_to_float(vr[(size_t)d * page_size]), acc[i]);
            }
        }
    }

    const float inv = l > 0.f ? 1.0f / l : 0.f;
    TO* orow = out + ((size_t)t * nq + h) * hd;
#pragma unroll
    for (int i = 0; i < ACC_REGS; ++i) {
        const int d = lane + HB_WAVE * i;
        if (d < hd) orow[d] = hb_from_float<TO>(acc[i] * inv);
    }
}

// q, out: [T, nq * hd]; keys [pages, nkv, page_size, hd], values [pages, nkv, hd, page_size];
// dtype covers q, cache and out.
extern "C" int hb_attention_plain(const void* q, const void* k_cache, const void* v_cache, void* out,
                                  int dtype, const int* positions, const int* seq_of, const int* slots,
                                  const int* page_table, int max_pages, int page_size, int T, int nq,
                                  int nkv, int hd, float scale, int window, hipStream_t stream) {
    HB_REQUIRE(T > 0 && nq > 0 && nkv > 0, "attention: empty input");
    HB_REQUIRE(nq % nkv == 0, "attention: %d query heads not divisible by %d kv heads", nq, nkv);
    HB_REQUIRE(hd > 0 && hd <= HB_MAX_HEAD_DIM, "attention: head_dim %d not in 1..%d", hd,
               HB_MAX_HEAD_DIM);
    HB_REQUIRE(page_size > 0 && window >= 0, "attention: bad page size or window");
    HB_REQUIRE(nq <= 65535, "attention: too many heads for the grid");
    dim3 grid(T, nq);
    if (dtype == HB_F32)
        attention_plain_kernel<float, float, float><<<grid, HB_WAVE, 0, stream>>>(
            (const float*)q, (const float*)k_cache, (const float*)v_cache, (float*)out, positions, seq_of,
            slots, page_table, max_pages, page_size, nq, nkv, hd, scale, window);
    else if (dtype == HB_BF16)
        attention_plain_kernel<bf16, bf16, bf16><<<grid, HB_WAVE, 0, stream>>>(
            (const bf16*)q, (const bf16*)k_cache, (const bf16*)v_cache, (bf16*)out, positions, seq_of,
            slots, page_table, max_pages, page_size, nq, nkv, hd, scale, window);
    else
        HB_REQUIRE(false, "attention: unknown dtype %d", dtype);
    HB_CHECK_LAUNCH("attention_plain");
    return 0;
}
