// bfloat16 attention over the paged cache on the gfx950 matrix cores.
//
// Cache layout: keys [page, kv head, 64 tokens, hd] (hd contiguous: the contraction of Q K^T),
// values transposed [page, kv head, hd, 64 tokens] (tokens contiguous: the contraction of P V).
// Both products are computed transposed with the 32x32x16 MFMA:
//   S^T[key, query] = K Q^T      first operand K rows, second operand Q rows
//   O^T[d,   query] = V^T P^T    first operand V^T rows, second operand P^T, which is S^T's
//                                own accumulator layout, so P never leaves the registers.
// A lane then owns one query column: the running maximum and sum of the online softmax are
// per-lane scalars (one exchange with the lane 32 apart). The 32 rows of a key block are
// assigned to keys in the order perm() below, which makes a lane's 8 values of one PV step
// 8 consecutive keys: V^T operands are single 16-byte reads.
//
// prefill: one workgroup = 32 consecutive tokens of one sequence x up to 4 query heads of one
//          kv head (one wave each); K and V^T pages go through a ring of two LDS stages once
//          for all of them, the keys a page ahead of the values.
// decode:  one wave = one sequence x one kv head x one range of pages, all query heads of the
//          group as columns; operands stream from global memory (each byte is used once);
//          partial (reference, sum, O) per range are merged by a second kernel in the fixed
//          order of the ranges. The kernel can also norm and rotate q and k and write the new
//          token's key and value itself.
// In xigh/herbert-rs the same sums are crates/backends/backend_common/src/generic_attention/prefill/kernel_f32.rs:39-113
// (prompts: causal by count, online softmax) and crates/backends/backend_common/src/attention_common.rs:20-124
// (decoding over a bfloat16 cache); the split of a long context into ranges whose partial (max, sum,
// output) a second kernel merges is crates/backends/backend_metal/shaders/attention_decode_flash.metal:30-198
// (tiles of 256 positions there), a key row shared by the query heads of its kv head as in
// crates/backends/backend_common/src/avx512_attn_dot8_bf16.S. The new key's norm, rotation and cache write inside the
// decode kernel: crates/backends/backend_metal/shaders/head_norm_rope_kv_append.metal:37-110.
#include "common.h"
#include <math.h>
#include <type_traits>

HB_MODULE_ERROR_SLOT()

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

#define PAGE 64
#define QTILE 32

// MFMA row rho (0..31) of a key block -> key within the block.
// rho = 16h + 8b + 4g + r  ->  16h + 8g + 4b + r  (h, b, g in {0,1}, r in 0..3)
__device__ __forceinline__ int perm(int rho) {
    return (rho & 16) | ((rho & 4) << 1) | ((rho & 8) >> 1) | (rho & 3);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// accumulator element i of lane group g2 of key block kb -> key within the page
__device__ __forceinline__ int acc_key(int kb, int g2, int i) { return kb * 32 + 16 * (i >> 3) + 8 * g2 + (i & 7); }

// One page of scores: mask, online-softmax update, P^T as MFMA operands.
// st[kb]: S^T accumulators (raw dot products). c = scale * log2(e).
// Keys k with lo <= page0 + k <= hi are visible; MASKED = false: the caller knows that all are.
// m is the reference of the exponents, not always the maximum: it is moved up (and the sums so
// far scaled by corr < 1) only when a score exceeds it by more than 8 / c, that is when a
// probability would exceed 2^8 times the largest so far; till then corr is 1 and the caller
// need not touch its sums. Any reference gives the same quotient in the end.
__device__ __forceinline__ float max_with_other_half(float v) {
    // lanes i and i ^ 32 exchange their values without a trip through LDS
    const unsigned u = __float_as_uint(v);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

#define RESCALE_LOG2 8.0f
template <bool MASKED>
__device__ __forceinline__ void softmax_page(f32x16 st[2], int g2, int page0, int lo, int hi, float c,
                                             float& m, float& l, float& corr, bf16x8 pb[2][2]) {
    float mx = -INFINITY;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            if (MASKED) {
                const int key = page0 + acc_key(kb, g2, i);
                st[kb][i] = (key >= lo && key <= hi) ? st[kb][i] : -INFINITY;
            }
            mx = fmaxf(mx, st[kb][i]);
        }
    mx = max_with_other_half(mx);
    corr = 1.0f;
    if ((mx - m) * c > RESCALE_LOG2 || m == -INFINITY) {       // (-inf) - (-inf) is NaN: compares false
        const float m_new = (mx == -INFINITY) ? m : mx;
        corr = (m == -INFINITY) ? 0.f : fast_exp2((m - m_new) * c);
        m = m_new;
    }
    const float mc = (m == -INFINITY) ? 0.f : m * c;
    float sum = 0.f;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const float p = fast_exp2(fmaf(st[kb][i], c, -mc));
            sum += p;
            pb[kb][i >> 3][i & 7] = (__bf16)p;
        }
    l = l * corr + sum;      // this lane's keys only; the two halves are added at the end
}

// oacc *= corr, unless corr is 1 in every lane
template <int NACC>
__device__ __forceinline__ void rescale(f32x16 (&oacc)[NACC], float corr) {
    if (__builtin_amdgcn_ballot_w64(corr != 1.0f) == 0) return;
#pragma unroll
    for (int d = 0; d < NACC; ++d)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[d][i] *= corr;
}

// The first half of softmax_page alone: mask, the page's largest score, the reference moved up if
// need be. Returns m * c (what is taken off the scaled scores), corr as softmax_page does.
template <bool MASKED>
__device__ __forceinline__ float softmax_reference(f32x16 st[2], int g2, int page0, int lo, int hi, float c,
                                                   float& m, float& corr) {
    float mx = -INFINITY;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            if (MASKED) {
                const int key = page0 + acc_key(kb, g2, i);
                st[kb][i] = (key >= lo && key <= hi) ? st[kb][i] : -INFINITY;
            }
            mx = fmaxf(mx, st[kb][i]);
        }
    mx = max_with_other_half(mx);
    corr = 1.0f;
    if ((mx - m) * c > RESCALE_LOG2 || m == -INFINITY) {
        const float m_new = (mx == -INFINITY) ? m : mx;
        corr = (m == -INFINITY) ? 0.f : fast_exp2((m - m_new) * c);
        m = m_new;
    }
    return (m == -INFINITY) ? 0.f : m * c;
}

// ----------------------------------------------------------------- prefill
// A read of 16 bytes from LDS that the compiler does not follow: it neither waits for it nor
// knows that it is in flight, so the caller waits by count (lds_wait<N>: at most N reads, in the
// order in which they were issued, may still be on their way) before the value is used. The
// compiler's own waits drain every read in flight (lgkmcnt(0)) each time a value is needed, the
// one issued a moment ago included; with three reads ahead of their products a wave of the
// prompt kernels then stood still for a read's whole way through LDS eleven times a page.
template <int BYTES_ON>
__device__ __forceinline__ bf16x8 lds_read_ahead(const bf16* p) {
    bf16x8 v;
    const uint32_t at = (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) bf16*)p;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(at), "n"(BYTES_ON));
    return v;
}
// (the value that is about to be used goes through the wait, so that its use cannot be moved before it)
template <int N>
__device__ __forceinline__ void lds_wait(bf16x8& arrived) {
    asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(arrived) : "n"(N));
}

// f(integral_constant<int, B>), ..., f(integral_constant<int, E - 1>): a loop whose index is a
// constant inside the body
template <int B, int E, class F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (B < E) {
        f(std::integral_constant<int, B>{});
        static_for<B + 1, E>(f);
    }
}

// What a lane needs to find its operands in the LDS stages of a page's keys and values.
struct PrefillLane {
    int c32, g2, krow, k_read[2], v_swz;
};

// The matrix products of one step of the prompt kernels, in the order in which they are issued:
// the scores of the next page S (HD / 8 of them: k-step j / 2 of key block j % 2) and this page's
// P V (four groups of 8 probabilities x HD / 32 blocks of the output). Between them go the
// exponentials, one group of 8 ahead of the P V products that use it, so that the vector units
// work in the shadow of the matrix cores within the wave itself: a wave issues in order, and a
// run of MFMAs followed by a run of exponentials would leave each unit idle in turn.
//   phase 0:        S[0, Q)                                 exp of group 0
//   phase g = 1..3: S[g Q, (g + 1) Q), P V of group g - 1   exp of group g
//   phase 4:        P V of group 3
// with Q = HD / 32. The LDS operand of a product is read AHEAD products before it is used.
// kst: the stage of the next page's keys; vst: the stage of this page's values. After the last
// page the scores "of the next" are worked out all the same, from whatever that stage holds,
// and never looked at: a second copy of the code without them costs more registers than a wave has.
template <int HD>
__device__ __forceinline__ void prefill_step_products(const bf16* kst, const bf16* vst, f32x16 (&st)[2],
                                                      f32x16 (&nxt)[2], f32x16 (&oacc)[HD / 32],
                                                      const bf16x8 (&qreg)[HD / 16], const PrefillLane& ln, float c,
                                                      float mc, float corr, float& l) {
    constexpr int Q = HD / 32, NM = 8 * Q, AHEAD = 3;
    const int c32 = ln.c32, g2 = ln.g2, krow = ln.krow, v_swz = ln.v_swz;
    // product n of the step: is it a score product, and which
    auto is_s = [](int n) { return n < Q || (n < 7 * Q && (n - Q) % (2 * Q) < Q); };
    auto s_index = [](int n) { return n < Q ? n : ((n - Q) / (2 * Q) + 1) * Q + (n - Q) % (2 * Q); };
    auto pv_group = [](int n) { return n < 7 * Q ? (n - Q) / (2 * Q) : 3; };
    auto pv_block = [](int n) { return n < 7 * Q ? (n - Q) % (2 * Q) - Q : n - 7 * Q; };
    constexpr int KRPB = 128 / HD > 0 ? 128 / HD : 1;
    // (an address is a lane's own part, shared by the two key blocks of a k-step and by the output
    // blocks of a group of probabilities, plus a constant that goes into the instruction)
    auto operand = [&](auto n_tag) -> bf16x8 {
        constexpr int n = decltype(n_tag)::value;
        if constexpr (is_s(n)) {
            constexpr int j = s_index(n), ks = j / 2, kb = j % 2;
            return lds_read_ahead<kb * 32 * HD * 2>(kst + krow * HD + (((2 * ks + g2) ^ ln.k_read[0]) * 8));
        } else {
            constexpr int g = pv_group(n), d = pv_block(n), kb = g >> 1, h2 = g & 1;
            return lds_read_ahead<d * 32 * PAGE * 2>(vst + c32 * PAGE + (((kb * 4 + h2 * 2 + g2) ^ v_swz) * 8));
        }
    };
    (void)KRPB;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int e = 0; e < 16; ++e) nxt[kb][e] = 0.f;
    bf16x8 ops[NM];
    bf16x8 pb[4];
    float sum = 0.f;
    // exponential e (0..7) of group g: element 8 * (g & 1) + e of key block g >> 1
    auto exponential = [&](int g, int e) {
        const float p = fast_exp2(fmaf(st[g >> 1][8 * (g & 1) + e], c, -mc));
        sum += p;
        pb[g][e] = (__bf16)p;
    };
    static_for<0, AHEAD>([&](auto t) { ops[decltype(t)::value] = operand(t); });
    static_for<0, NM>([&](auto t) {
        constexpr int n = decltype(t)::value;
        if constexpr (n + AHEAD < NM) ops[n + AHEAD] = operand(std::integral_constant<int, n + AHEAD>{});
        // the reads behind product n's own may still be on their way: AHEAD of them, fewer at the end
        lds_wait<(n + AHEAD < NM ? AHEAD : NM - 1 - n)>(ops[n]);
        if constexpr (is_s(n)) {
            constexpr int j = s_index(n);
            nxt[j % 2] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ops[n], qreg[j / 2], nxt[j % 2], 0, 0, 0);
        } else {
            constexpr int d = pv_block(n);
            oacc[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ops[n], pb[pv_group(n)], oacc[d], 0, 0, 0);
        }
        // the exponentials that go with this product: those of phase g are dealt out over the
        // phase's products (phase 0 has Q of them, the others 2 Q)
        if constexpr (n < 7 * Q) {
            constexpr int g = n < Q ? 0 : (n - Q) / (2 * Q) + 1;
            constexpr int in_phase = n < Q ? n : (n - Q) % (2 * Q), of = n < Q ? Q : 2 * Q;
#pragma unroll
            for (int e = in_phase * 8 / of; e < (in_phase + 1) * 8 / of; ++e) exponential(g, e);
        }
        __builtin_amdgcn_sched_barrier(0);
    });
    l = l * corr + sum;      // this lane's keys only; the two halves are added at the end
}

// A workgroup: 32 queries x up to 4 query heads of one kv head, by eight waves in two groups of
// four (a wave a head in each group). The groups take the tile's pages in turn, the first the
// even ones and the second the odd ones, each with a reference, a sum and an output of its
// own, which are added up through LDS at the end: the tile with the most pages, which decides
// how long a prompt of a few thousand tokens takes, is done in half as many steps, and a CU
// holds one workgroup whose eight waves (two a SIMD) are busy from its first page to its last.
// Each group's pages go from global memory straight into a ring of two LDS stages of its own,
// the next page's loads in flight while this page is worked on. Rows lie unpadded; the
// 16-byte chunk c of row r sits at chunk c ^ (r / rows in 256 bytes), so that the operand
// reads of 16 rows at one chunk fall into 16 different bank groups.
// Workgroups are numbered by falling work (the host sorts the tiles): a CU that is done takes
// the heaviest tile left.
template <int HD>
__global__ void __launch_bounds__(512, 1)
attn_prefill_kernel(const bf16* __restrict__ q, const bf16* __restrict__ k_cache,
                    const bf16* __restrict__ v_cache, bf16* __restrict__ out,
                    const int* __restrict__ tile_seq, const int* __restrict__ tile_row0,
                    const int* __restrict__ tile_rows, const int* __restrict__ positions,
                    const int* __restrict__ slots, const int* __restrict__ page_table, int max_pages, int nq,
                    int nkv, float c, int window, int per_tile) {
    constexpr int KCH = HD / 8;                   // 16-byte chunks of a key row
    constexpr int KRPB = 128 / HD > 0 ? 128 / HD : 1;   // key rows in 256 bytes
    constexpr int KROWS = 512 / HD;               // key rows a load instruction brings (1 KB)
    constexpr int LOADS = HD / 32;                // a wave's load instructions for the keys of a page; as many for the values
    constexpr int STAGE = PAGE * HD;              // elements of one stage of keys, or of values
    // The LDS is the launch's (extern), not arrays of this kernel: for an array of its own the
    // compiler knows which loads-to-LDS may alias a read and waits for every load in flight
    // (s_waitcnt vmcnt(0)) before the first read that follows, which undoes the ring: the loads of
    // the next pages would be waited for at once. What has to have landed is waited for by hand.
    extern __shared__ __attribute__((aligned(1024))) bf16 attn_lds[];     // [group][keys [2][STAGE], values [2][STAGE]]

    const int w = blockIdx.x;
    const int tile = w / per_tile, y = w % per_tile;
    const int G = nq / nkv;
    const int chunks = (G + 3) / 4;
    const int kvh = y / chunks;
    const int chunk = y % chunks;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave8 = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int grp = wave8 >> 2, wave = wave8 & 3;
    bf16* const Ks = attn_lds + grp * 4 * STAGE;
    bf16* const Vs = Ks + 2 * STAGE;
    const int c32 = lane & 31, g2 = lane >> 5;
    const int head_in_group = chunk * 4 + wave;
    const bool active = head_in_group < G;
    const int h = kvh * G + (active ? head_in_group : G - 1);

    const int row0 = tile_row0[tile];
    const int rows = tile_rows[tile];
    const int slot = slots[tile_seq[tile]];
    const int* pt = page_table + (size_t)slot * max_pages;
    const int pos0 = positions[row0];
    const int my_row = c32 < rows ? c32 : rows - 1;
    const int pos_q = pos0 + my_row;
    const int lo_q = (window > 0 && pos_q + 1 > window) ? pos_q + 1 - window : 0;
    const int hi_tile = pos0 + rows - 1;                                     // last visible key
    const int lo_tile = (window > 0 && pos0 + 1 > window) ? pos0 + 1 - window : 0;
    const int first_page = lo_tile / PAGE, last_page = hi_tile / PAGE;
    // this group's pages: first_page + grp, + 2, ...; the first group has as many as the second or one more
    const int steps = (last_page - first_page) / 2 + 1;                      // of the first group: every wave loops so often
    const int mine = last_page - first_page - grp >= 0 ? (last_page - first_page - grp) / 2 + 1 : 0;
    auto page_of = [&](int i) { return first_page + grp + 2 * i; };

    // this lane's part of the loads of a page: element offsets within the page's keys and values
    int k_off[LOADS], v_off[LOADS];
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
        const int instr = wave * LOADS + i;
        const int kr = instr * KROWS + lane / KCH;
        k_off[i] = kr * HD + (((lane % KCH) ^ ((kr / KRPB) % KCH)) * 8);
        const int vr = instr * 8 + lane / 8;
        v_off[i] = vr * PAGE + (((lane & 7) ^ ((vr >> 1) & 7)) * 8);
    }
    auto issue_keys = [&](int i, int stage) {
        const bf16* kp = k_cache + ((size_t)pt[page_of(i)] * nkv + kvh) * PAGE * HD;
#pragma unroll
        for (int j = 0; j < LOADS; ++j) hb_load_to_lds(kp + k_off[j], Ks + stage * STAGE + (wave * LOADS + j) * 512);
    };
    auto issue_values = [&](int i, int stage) {
        const bf16* vp = v_cache + ((size_t)pt[page_of(i)] * nkv + kvh) * HD * PAGE;
#pragma unroll
        for (int j = 0; j < LOADS; ++j) hb_load_to_lds(vp + v_off[j], Vs + stage * STAGE + (wave * LOADS + j) * 512);
    };
    // The keys run one page ahead of the values: the scores of the group's next page are on the
    // matrix cores while the softmax of this one runs on the vector units.
    if (mine > 0) {
        issue_keys(0, 0);
        issue_values(0, 0);
    }
    if (mine > 1) issue_keys(1, 1);

    bf16x8 qreg[HD / 16];
    {
        const bf16* qrow = q + ((size_t)(row0 + my_row) * nq + h) * HD + g2 * 8;
#pragma unroll
        for (int s = 0; s < HD / 16; ++s) qreg[s] = *(const bf16x8*)(qrow + s * 16);
    }

    f32x16 oacc[HD / 32];
#pragma unroll
    for (int d = 0; d < HD / 32; ++d)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[d][i] = 0.f;
    float m = -INFINITY, l = 0.f;

    const int krow = perm(c32);
    int k_read[2];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) k_read[kb] = ((kb * 32 + krow) / KRPB) % KCH;
    const int v_swz = (c32 >> 1) & 7;            // of rows d * 32 + c32
    const PrefillLane ln = {c32, g2, krow, {k_read[0], k_read[1]}, v_swz};
    // raw scores of the page in a key stage; the two key blocks alternate, so that no MFMA waits
    // for the one before it
    auto scores = [&](int stage, f32x16 (&st)[2]) {
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int i = 0; i < 16; ++i) st[kb][i] = 0.f;
#pragma unroll
        for (int s = 0; s < HD / 16; ++s)
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                const bf16x8 ka = *(const bf16x8*)(Ks + stage * STAGE + (kb * 32 + krow) * HD + (((2 * s + g2) ^ k_read[kb]) * 8));
                st[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka, qreg[s], st[kb], 0, 0, 0);
            }
    };
    // One step of the group: its page i, whose scores are in `st`; the scores of page i + 1 go to `nxt`.
    auto step = [&](auto parity_tag, int i, f32x16 (&st)[2], f32x16 (&nxt)[2]) {
        // landed, for every wave after the barrier: the values of this page and the keys of the
        // next; and nobody reads any more the key stage of this page (its scores are done) nor
        // the value stage of the page before, which the next loads fill
        hb_wait_vmcnt<0>();
        hb_workgroup_barrier();
        if (i + 2 < mine) issue_keys(i + 2, i & 1);
        if (i + 1 < mine) issue_values(i + 1, (i + 1) & 1);
        if (!active || i >= mine) return;
        float corr, mc;
        // a page that every query of the tile sees whole needs no mask
        const int page0 = page_of(i) * PAGE;
        if (page0 + PAGE - 1 <= pos0 && (window == 0 || page0 >= hi_tile + 1 - window))
            mc = softmax_reference<false>(st, g2, page0, lo_q, pos_q, c, m, corr);
        else
            mc = softmax_reference<true>(st, g2, page0, lo_q, pos_q, c, m, corr);
        rescale(oacc, corr);          // rarely: the reference moves lazily
        // (the parity of the step is known where the code is written out, twice a round: the stage
        // of an operand is then a constant offset of its read and costs no register)
        constexpr int PAR = decltype(parity_tag)::value;
        prefill_step_products<HD>(Ks + ((PAR + 1) & 1) * STAGE, Vs + PAR * STAGE, st, nxt, oacc, qreg, ln, c, mc, corr, l);
    };
    hb_wait_vmcnt<0>();
    hb_workgroup_barrier();
    f32x16 sa[2], sb[2];
    if (active && mine > 0) scores(0, sa);
    for (int i = 0; i < steps; i += 2) {           // two steps a round: the scores change places, nothing is copied
        step(std::integral_constant<int, 0>{}, i, sa, sb);
        if (i + 1 < steps) step(std::integral_constant<int, 1>{}, i + 1, sb, sa);
    }
    // The second group hands over what it has: reference, sum and output of every lane, through
    // the LDS that held the rings (nobody reads those any more after the barrier, and no load
    // is in flight), [wave][value][lane].
    hb_wait_vmcnt<0>();
    hb_workgroup_barrier();
    float* const hand = (float*)attn_lds + (size_t)wave * (HD / 2 + 2) * 64 + lane;
    if (grp == 1 && active) {
        hand[0] = m;
        hand[64] = l;
#pragma unroll
        for (int d = 0; d < HD / 32; ++d)
#pragma unroll
            for (int i = 0; i < 16; ++i) hand[(2 + d * 16 + i) * 64] = oacc[d][i];
    }
    __syncthreads();
    if (grp == 1 || !active || c32 >= rows) return;
    {
        const float m1 = hand[0], l1 = hand[64];
        const float mm = fmaxf(m, m1);
        // (a group without a visible key has the reference -inf, the sum 0 and the output 0)
        const float a0 = m == -INFINITY ? 0.f : fast_exp2((m - mm) * c);
        const float a1 = m1 == -INFINITY ? 0.f : fast_exp2((m1 - mm) * c);
        l = l * a0 + l1 * a1;
#pragma unroll
        for (int d = 0; d < HD / 32; ++d)
#pragma unroll
            for (int i = 0; i < 16; ++i) oacc[d][i] = oacc[d][i] * a0 + hand[(2 + d * 16 + i) * 64] * a1;
    }
    l += __shfl_xor(l, 32, 64);
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    bf16* orow = out + ((size_t)(row0 + c32) * nq + h) * HD;
#pragma unroll
    for (int d = 0; d < HD / 32; ++d)
#pragma unroll
        for (int qd = 0; qd < 4; ++qd) {
            bf16x4 v;
#pragma unroll
            for (int r = 0; r < 4; ++r) v[r] = (__bf16)(oacc[d][4 * qd + r] * inv);
            *(bf16x4*)(orow + d * 32 + 8 * qd + 4 * g2) = v;
        }
}

// The prompt kernel for long prompts (many tiles, all of them long): a workgroup is 64 consecutive
// tokens x up to 4 query heads of one kv head; its eight waves are two halves of 32 tokens (a wave
// a head in each) that share the pages: one ring of three LDS stages for the keys and one for the
// values, every page loaded once for both halves, so that half as many bytes go into LDS for a
// product and a page's loads have two steps to land instead of one (the kernel above waits for
// its loads for a third of its time). No merge at the end: a half owns its rows.
// Every wave issues the same number of loads in every step (past the last page: that page again,
// into a stage nobody reads any more), so that the wait before the barrier can count: all but
// the loads of the step before have landed.
template <int HD>
__global__ void __launch_bounds__(512, 1)
attn_prefill_long_kernel(const bf16* __restrict__ q, const bf16* __restrict__ k_cache,
                         const bf16* __restrict__ v_cache, bf16* __restrict__ out,
                         const int* __restrict__ tile_seq, const int* __restrict__ tile_row0,
                         const int* __restrict__ tile_rows, const int* __restrict__ positions,
                         const int* __restrict__ slots, const int* __restrict__ page_table, int max_pages,
                         int nq, int nkv, float c, int window, int per_tile) {
    constexpr int KCH = HD / 8;
    constexpr int KRPB = 128 / HD > 0 ? 128 / HD : 1;
    constexpr int KROWS = 512 / HD;
    constexpr int INSTRS = HD / 8;                // load instructions (1 KB each) for the keys of a page; as many for the values
    constexpr int PL = INSTRS >= 8 ? INSTRS / 8 : 1;   // of which a wave issues (with fewer than 8, the first waves one each)
    constexpr int STAGE = PAGE * HD;
    extern __shared__ __attribute__((aligned(1024))) bf16 attn_lds[];     // keys [3][STAGE], values [3][STAGE]
    bf16* const Ks = attn_lds;
    bf16* const Vs = attn_lds + 3 * STAGE;

    const int w = blockIdx.x;
    const int tile = w / per_tile, y = w % per_tile;
    const int G = nq / nkv;
    const int chunks = (G + 3) / 4;
    const int kvh = y / chunks;
    const int chunk = y % chunks;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave8 = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int half = wave8 >> 2, wave = wave8 & 3;
    const int c32 = lane & 31, g2 = lane >> 5;
    const int head_in_group = chunk * 4 + wave;

    const int tile_row = tile_row0[tile], tile_n = tile_rows[tile];          // up to 64 rows
    const int rows = tile_n - 32 * half < 32 ? tile_n - 32 * half : 32;      // of this half; <= 0: it has none
    const bool active = head_in_group < G && rows > 0;
    const int h = kvh * G + (head_in_group < G ? head_in_group : G - 1);
    const int row0 = tile_row + (rows > 0 ? 32 * half : 0);
    const int slot = slots[tile_seq[tile]];
    const int* pt = page_table + (size_t)slot * max_pages;
    const int tile_pos0 = positions[tile_row];
    const int pos0 = tile_pos0 + (rows > 0 ? 32 * half : 0);
    const int my_row = rows > 0 ? (c32 < rows ? c32 : rows - 1) : 0;
    const int pos_q = pos0 + my_row;
    const int lo_q = (window > 0 && pos_q + 1 > window) ? pos_q + 1 - window : 0;
    const int hi_half = pos0 + (rows > 0 ? rows : 1) - 1;                     // last key this half sees
    // the workgroup's pages: from the first a row of the tile sees to the last
    const int lo_tile = (window > 0 && tile_pos0 + 1 > window) ? tile_pos0 + 1 - window : 0;
    const int first_page = lo_tile / PAGE, last_page = (tile_pos0 + tile_n - 1) / PAGE;
    const int steps = last_page - first_page + 1;
    const int mine = active ? hi_half / PAGE - first_page + 1 : 0;            // this half's steps: pages up to its own last
    auto page_of = [&](int i) { return first_page + (i < steps ? i : steps - 1); };   // past the end: the last page again

    int k_off[PL], v_off[PL];
    const bool loads = INSTRS >= 8 || wave8 < INSTRS;
#pragma unroll
    for (int i = 0; i < PL; ++i) {
        const int instr = (INSTRS >= 8 ? wave8 * PL + i : wave8) % INSTRS;
        const int kr = instr * KROWS + lane / KCH;
        k_off[i] = kr * HD + (((lane % KCH) ^ ((kr / KRPB) % KCH)) * 8);
        const int vr = instr * 8 + lane / 8;
        v_off[i] = vr * PAGE + (((lane & 7) ^ ((vr >> 1) & 7)) * 8);
    }
    auto issue_keys = [&](int i) {
        if (!loads) return;
        const bf16* kp = k_cache + ((size_t)pt[page_of(i)] * nkv + kvh) * PAGE * HD;
#pragma unroll
        for (int j = 0; j < PL; ++j) {
            const int instr = (INSTRS >= 8 ? wave8 * PL + j : wave8) % INSTRS;
            hb_load_to_lds(kp + k_off[j], Ks + (i % 3) * STAGE + instr * 512);
        }
    };
    auto issue_values = [&](int i) {
        if (!loads) return;
        const bf16* vp = v_cache + ((size_t)pt[page_of(i)] * nkv + kvh) * HD * PAGE;
#pragma unroll
        for (int j = 0; j < PL; ++j) {
            const int instr = (INSTRS >= 8 ? wave8 * PL + j : wave8) % INSTRS;
            hb_load_to_lds(vp + v_off[j], Vs + (i % 3) * STAGE + instr * 512);
        }
    };
    // in flight before the first step: the keys of pages 0, 1, 2 and the values of pages 0, 1; the
    // last two of these five are what a step leaves in flight
    issue_keys(0);
    issue_values(0);
    issue_keys(1);
    issue_values(1);
    issue_keys(2);

    bf16x8 qreg[HD / 16];
    {
        const bf16* qrow = q + ((size_t)(row0 + my_row) * nq + h) * HD + g2 * 8;
#pragma unroll
        for (int s2 = 0; s2 < HD / 16; ++s2) qreg[s2] = *(const bf16x8*)(qrow + s2 * 16);
    }
    f32x16 oacc[HD / 32];
#pragma unroll
    for (int d = 0; d < HD / 32; ++d)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[d][i] = 0.f;
    float m = -INFINITY, l = 0.f;
    const int krow = perm(c32);
    PrefillLane ln;
    ln.c32 = c32;
    ln.g2 = g2;
    ln.krow = krow;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) ln.k_read[kb] = ((kb * 32 + krow) / KRPB) % KCH;
    ln.v_swz = (c32 >> 1) & 7;

    auto step = [&](int i, f32x16 (&st)[2], f32x16 (&nxt)[2]) {
        // landed, for every wave after the barrier: all but what the step before asked for, that is
        // the keys of page i + 1 and the values of page i; and nobody reads any more the stages that
        // this step's loads fill (the keys of page i, the values of page i - 1)
        if (loads) hb_wait_vmcnt<2 * PL>();
        hb_workgroup_barrier();
        issue_values(i + 2);
        issue_keys(i + 3);
        if (i >= mine) return;
        float corr, mc;
        const int page0 = page_of(i) * PAGE;
        if (page0 + PAGE - 1 <= pos0 && (window == 0 || page0 >= hi_half + 1 - window))
            mc = softmax_reference<false>(st, g2, page0, lo_q, pos_q, c, m, corr);
        else
            mc = softmax_reference<true>(st, g2, page0, lo_q, pos_q, c, m, corr);
        rescale(oacc, corr);
        prefill_step_products<HD>(Ks + ((i + 1) % 3) * STAGE, Vs + (i % 3) * STAGE, st, nxt, oacc, qreg, ln, c, mc,
                                  corr, l);
    };
    // the first page's scores: its keys are the oldest of the five sets of loads (and of the
    // query's own loads behind them)
    if (loads) hb_wait_vmcnt<3 * PL>();
    hb_workgroup_barrier();
    f32x16 sa[2], sb[2];
    if (mine > 0) {
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int i = 0; i < 16; ++i) sa[kb][i] = 0.f;
#pragma unroll
        for (int s2 = 0; s2 < HD / 16; ++s2)
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                const bf16x8 ka = *(const bf16x8*)(Ks + (kb * 32 + krow) * HD + (((2 * s2 + g2) ^ ln.k_read[kb]) * 8));
                sa[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka, qreg[s2], sa[kb], 0, 0, 0);
            }
    }
    for (int i = 0; i < steps; i += 2) {
        step(i, sa, sb);
        if (i + 1 < steps) step(i + 1, sb, sa);
    }
    hb_wait_vmcnt<0>();          // nothing of this workgroup's is in flight when it ends
    if (!active || c32 >= rows) return;
    l += __shfl_xor(l, 32, 64);
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    bf16* orow = out + ((size_t)(row0 + c32) * nq + h) * HD;
#pragma unroll
    for (int d = 0; d < HD / 32; ++d)
#pragma unroll
        for (int qd = 0; qd < 4; ++qd) {
            bf16x4 v;
#pragma unroll
            for (int r = 0; r < 4; ++r) v[r] = (__bf16)(oacc[d][4 * qd + r] * inv);
            *(bf16x4*)(orow + d * 32 + 8 * qd + 4 * g2) = v;
        }
}

// ------------------------------------------------------------------ decode
// partial_o [B, nq, splits, HD] float, partial_ml [B, nq, splits, 2] float (max, sum).
// FUSED: q is not given; the kernel takes the float32 projection rows qkv [B, (nq + 2 nkv) HD]
// instead and does the per-head RMSNorm (if weights are given) and the rotation (if tables are
// given, over the whole head) itself: every wave for its query heads, and the one wave whose
// range holds the new position also for the new key and value, which it writes to the pages
// before it reads them (write_kv == 0: the keys and values are another layer's).
// QS > 1: the projection was cut into QS slices of K whose sums lie slice_stride floats apart
// behind qkv; the kernel adds them up in their order as it loads them (no kernel of its own does).
struct DecodeFusion {
    const float* qkv;
    const float* q_norm_w;
    const float* k_norm_w;
    const float* cos_t;
    const float* sin_t;
    float eps;
    int write_kv;
    size_t slice_stride;
};

template <int HD, bool FUSED, int QS = 1>
__global__ void __launch_bounds__(64)
attn_decode_kernel(const bf16* __restrict__ q, bf16* __restrict__ k_cache, bf16* __restrict__ v_cache,
                   float* __restrict__ partial_o, float* __restrict__ partial_ml,
                   const int* __restrict__ context_lens, const int* __restrict__ slots,
                   const int* __restrict__ page_table, int max_pages, int nq, int nkv, float c, int window,
                   int pages_per_split, DecodeFusion fu, bf16* __restrict__ out,
                   const int* __restrict__ ranges, int n_seqs) {
    // ranges == null: the grid is (sequence, kv head, range), every sequence cut into gridDim.z
    // ranges of pages_per_split pages (those past a sequence's end hold nothing).
    // ranges != null (sequences of unequal lengths): the grid is (1, kv head, item);
    // ranges[0 .. n_seqs] count the ranges of the sequences before each one, ranges[n_seqs + 1] is
    // the pages of a range: item i is range i - ranges[b] of the sequence b whose count it falls
    // into, and items from ranges[n_seqs] on are nothing. The partial results are then laid out
    // [head, item]: those of one sequence and head lie side by side.
    const int kvh = blockIdx.y, splits = gridDim.z;
    const int lane = threadIdx.x, c32 = lane & 31, g2 = lane >> 5;
    int b = blockIdx.x, split = blockIdx.z;
    if (ranges) {
        const int item = blockIdx.z;
        b = 0;                                              // sequences wholly before the item
        for (int first = 0; first < n_seqs; first += 64) {
            const int upto = first + lane < n_seqs ? ranges[first + lane + 1] : 0x7fffffff;
            b += __popcll(__ballot(upto <= item));
        }
        b = __builtin_amdgcn_readfirstlane(b);
        if (b >= n_seqs) return;
        split = item - ranges[b];
        pages_per_split = ranges[n_seqs + 1];
    }
    const int G = nq / nkv;
    const int ctx = context_lens[b];                 // keys 0 .. ctx-1; the query sits at ctx-1
    const int hi = ctx - 1;
    const int lo = (window > 0 && ctx > window) ? ctx - window : 0;
    const int first_page = lo / PAGE + split * pages_per_split;
    int last_page = first_page + pages_per_split - 1;
    if (last_page > hi / PAGE) last_page = hi / PAGE;
    const int* pt = page_table + (size_t)slots[b] * max_pages;
    const int head = kvh * G + (c32 < G ? c32 : G - 1);

    constexpr int HALF = HD / 2;
    // k of the MFMA steps: step s, lane group g2, element j  <->  d = g2 * HD/2 + s * 8 + j,
    // so a lane reads one contiguous half row of K
    bf16x8 qreg[HD / 16];
    if (!FUSED) {
        const bf16* qrow = q + ((size_t)b * nq + head) * HD + g2 * HALF;
#pragma unroll
        for (int s = 0; s < HD / 16; ++s) qreg[s] = *(const bf16x8*)(qrow + s * 8);
    }

    // FUSED: lane -> the pair of elements (j, j + HD/2) of head `sub` of each round of 64 / (HD/2)
    // heads. What the norm and the rotation need is loaded before the first page's operands, so
    // that it arrives first.
    constexpr int PER = 64 / HALF;                 // heads a round of the wave covers
    constexpr int PRE = 4;                         // rounds whose inputs are loaded ahead
    const int j = lane % HALF, sub = lane / HALF;
    const int hp = hi / PAGE;
    const bool writer = FUSED && fu.write_kv && hp >= first_page && hp < first_page + pages_per_split;
    float cs = 1.f, sn = 0.f, qw0 = 1.f, qw1 = 1.f, kw0 = 1.f, kw1 = 1.f;
    float xq0[PRE], xq1[PRE], k0 = 0.f, k1 = 0.f, v0 = 0.f, v1 = 0.f;
    int new_page = 0;
    const float* qin = nullptr;
    if (FUSED) {
        const float* row = fu.qkv + (size_t)b * (nq + 2 * nkv) * HD;
        qin = row + (size_t)kvh * G * HD;
        if (fu.cos_t) {
            cs = fu.cos_t[(size_t)hi * HALF + j];
            sn = fu.sin_t[(size_t)hi * HALF + j];
        }
        if (fu.q_norm_w) {
            qw0 = fu.q_norm_w[j];
            qw1 = fu.q_norm_w[j + HALF];
        }
        // (all slices of a value are asked for together and added in their order)
        auto summed = [&](const float* p) {
            float part[QS];
#pragma unroll
            for (int i = 0; i < QS; ++i) part[i] = p[(size_t)i * fu.slice_stride];
            float sum = part[0];
#pragma unroll
            for (int i = 1; i < QS; ++i) sum += part[i];
            return sum;
        };
#pragma unroll
        for (int it = 0; it < PRE; ++it) {
            const int hl = it * PER + sub < G ? it * PER + sub : G - 1;
            xq0[it] = summed(qin + hl * HD + j);
            xq1[it] = summed(qin + hl * HD + j + HALF);
        }
        if (writer) {
            const float* kin = row + (size_t)(nq + kvh) * HD;
            const float* vin = row + (size_t)(nq + nkv + kvh) * HD;
            k0 = summed(kin + j);
            k1 = summed(kin + j + HALF);
            v0 = summed(vin + j);
            v1 = summed(vin + j + HALF);
            if (fu.k_norm_w) {
                kw0 = fu.k_norm_w[j];
                kw1 = fu.k_norm_w[j + HALF];
            }
            new_page = pt[hp];
        }
    }
    f32x16 oacc[HD / 32];
#pragma unroll
    for (int d = 0; d < HD / 32; ++d)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[d][i] = 0.f;
    float m = -INFINITY, l = 0.f;
    const int krow = perm(c32);

    // The loads of the next page go out as soon as the registers of the current one are free:
    // keys right after Q K^T, values right after P V, so that memory works while the wave computes.
    bf16x8 ka[2][HD / 16];
    bf16x8 va[HD / 32][2][2];
#define LOAD_K(PAGE_IDX)                                                                     \
    {                                                                                        \
        const bf16* kp = k_cache + ((size_t)pt[PAGE_IDX] * nkv + kvh) * PAGE * HD + g2 * (HD / 2); \
        _Pragma("unroll") for (int kb = 0; kb < 2; ++kb)                                     \
            _Pragma("unroll") for (int s = 0; s < HD / 16; ++s)                              \
                ka[kb][s] = *(const bf16x8*)(kp + (size_t)(kb * 32 + krow) * HD + s * 8);    \
    }
#define LOAD_V(PAGE_IDX)                                                                     \
    {                                                                                        \
        const bf16* vp = v_cache + ((size_t)pt[PAGE_IDX] * nkv + kvh) * HD * PAGE + g2 * 8;  \
        _Pragma("unroll") for (int d = 0; d < HD / 32; ++d)                                  \
            _Pragma("unroll") for (int kb = 0; kb < 2; ++kb)                                 \
                _Pragma("unroll") for (int h2 = 0; h2 < 2; ++h2)                             \
                    va[d][kb][h2] = *(const bf16x8*)(vp + (size_t)(d * 32 + c32) * PAGE + kb * 32 + h2 * 16); \
    }
    __shared__ __attribute__((aligned(16))) bf16 qs[FUSED ? 32 * HD : 8];
    // norm and rotation of the new key and of the query heads; the key and the value go to the pages,
    // the queries to LDS, from where each lane takes its operand
    auto prologue = [&]() {
        if (writer) {
            float ss = k0 * k0 + k1 * k1;
#pragma unroll
            for (int off = HALF / 2; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
            if (fu.k_norm_w) {
                const float inv = 1.0f / sqrtf(ss / (float)HD + fu.eps);
                k0 = k0 * inv * kw0;
                k1 = k1 * inv * kw1;
            }
            const float r0 = k0 * cs - k1 * sn, r1 = k0 * sn + k1 * cs;
            if (sub == 0) {
                const int in_page = hi % PAGE;
                bf16* kdst = k_cache + (((size_t)new_page * nkv + kvh) * PAGE + in_page) * HD;
                kdst[j] = hb_from_float<bf16>(r0);
                kdst[j + HALF] = hb_from_float<bf16>(r1);
                bf16* vdst = v_cache + ((size_t)new_page * nkv + kvh) * HD * PAGE + in_page;
                vdst[(size_t)j * PAGE] = hb_from_float<bf16>(v0);
                vdst[(size_t)(j + HALF) * PAGE] = hb_from_float<bf16>(v1);
            }
            __threadfence_block();      // this wave's later loads of that page see what it has just written
        }
        auto finish_head = [&](int hl, float x0, float x1) {
            if (fu.q_norm_w) {
                float ss = x0 * x0 + x1 * x1;
#pragma unroll
                for (int off = HALF / 2; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
                const float inv = 1.0f / sqrtf(ss / (float)HD + fu.eps);
                x0 = x0 * inv * qw0;
                x1 = x1 * inv * qw1;
            }
            if (hl < G) {
                qs[hl * HD + j] = hb_from_float<bf16>(x0 * cs - x1 * sn);
                qs[hl * HD + j + HALF] = hb_from_float<bf16>(x0 * sn + x1 * cs);
            }
        };
#pragma unroll
        for (int it = 0; it < PRE; ++it)
            if (it * PER < G) finish_head(it * PER + sub, xq0[it], xq1[it]);
        for (int it = PRE; it * PER < G; ++it) {
            const int hl = it * PER + sub;
            const int hs = hl < G ? hl : G - 1;
            float x0 = 0.f, x1 = 0.f;
#pragma unroll
            for (int i = 0; i < QS; ++i) {
                x0 += qin[(size_t)i * fu.slice_stride + hs * HD + j];
                x1 += qin[(size_t)i * fu.slice_stride + hs * HD + j + HALF];
            }
            finish_head(hl, x0, x1);
        }
    };
    // The first page's operands go out before that work, so that it hides their way from memory,
    // unless this wave has yet to write the new key into that very page. (Two copies of the code:
    // each then knows how many loads are in flight behind the small ones it waits for.)
    if (!FUSED) {
        if (first_page <= last_page) {
            LOAD_K(first_page)
            LOAD_V(first_page)
        }
    } else if (first_page <= last_page && !(writer && first_page == hp)) {
        LOAD_K(first_page)
        LOAD_V(first_page)
        prologue();
    } else {
        prologue();
        if (first_page <= last_page) {
            LOAD_K(first_page)
            LOAD_V(first_page)
        }
    }
    if (FUSED) {
        __syncthreads();
        const bf16* qrow = qs + (c32 < G ? c32 : G - 1) * HD + g2 * HALF;
#pragma unroll
        for (int s2 = 0; s2 < HD / 16; ++s2) qreg[s2] = *(const bf16x8*)(qrow + s2 * 8);
    }
    for (int page_idx = first_page; page_idx <= last_page; ++page_idx) {
        f32x16 st[2];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
            for (int i = 0; i < 16; ++i) st[kb][i] = 0.f;
#pragma unroll
            for (int s = 0; s < HD / 16; ++s)
                st[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka[kb][s], qreg[s], st[kb], 0, 0, 0);
        }
        if (page_idx < last_page) LOAD_K(page_idx + 1)
        float corr;
        bf16x8 pb[2][2];
        if (page_idx * PAGE >= lo && page_idx * PAGE + PAGE - 1 <= hi)
            softmax_page<false>(st, g2, page_idx * PAGE, lo, hi, c, m, l, corr, pb);
        else
            softmax_page<true>(st, g2, page_idx * PAGE, lo, hi, c, m, l, corr, pb);
        rescale(oacc, corr);
#pragma unroll
        for (int d = 0; d < HD / 32; ++d) {
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int h2 = 0; h2 < 2; ++h2)
                    oacc[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va[d][kb][h2], pb[kb][h2], oacc[d], 0, 0, 0);
        }
        if (page_idx < last_page) LOAD_V(page_idx + 1)
    }
#undef LOAD_K
#undef LOAD_V
    l += __shfl_xor(l, 32, 64);
    if (out) {
        // one range a sequence: nothing to merge, the output is O / l (zeros if no key was visible)
        if (c32 < G) {
            const float inv = l > 0.f ? 1.0f / l : 0.f;
            bf16* dst = out + ((size_t)b * nq + kvh * G + c32) * HD;
#pragma unroll
            for (int d = 0; d < HD / 32; ++d)
#pragma unroll
                for (int qd = 0; qd < 4; ++qd) {
                    bf16x4 v;
#pragma unroll
                    for (int j = 0; j < 4; ++j) v[j] = (__bf16)(oacc[d][4 * qd + j] * inv);
                    *(bf16x4*)((__bf16*)dst + d * 32 + 8 * qd + 4 * g2) = v;
                }
        }
        return;
    }
    if (c32 < G) {
        const size_t base = ranges ? (size_t)(kvh * G + c32) * splits + blockIdx.z
                                   : ((size_t)b * nq + kvh * G + c32) * splits + split;
        if (g2 == 0) {
            partial_ml[base * 2] = m;        // -inf when this range held no visible key
            partial_ml[base * 2 + 1] = l;
        }
        float* po = partial_o + base * HD;
#pragma unroll
        for (int d = 0; d < HD / 32; ++d)
#pragma unroll
            for (int qd = 0; qd < 4; ++qd) {
                f32x4 v = {oacc[d][4 * qd], oacc[d][4 * qd + 1], oacc[d][4 * qd + 2], oacc[d][4 * qd + 3]};
                *(f32x4*)(po + d * 32 + 8 * qd + 4 * g2) = v;
            }
    }
}

// Merge the ranges of one (sequence, head), in the order of the ranges:
//   out = sum_s 2^((m_s - M) c) O_s / sum_s 2^((m_s - M) c) l_s.
// One wave per (sequence, head). A kernel of its own: the partial results of waves on other
// XCDs are visible at a kernel boundary without any fence that would write back an L2.
template <int HD>
__global__ void __launch_bounds__(256)
attn_decode_merge_kernel(const float* __restrict__ partial_o, const float* __restrict__ partial_ml,
                         bf16* __restrict__ out, int splits, float c, const int* __restrict__ ranges, int nq) {
    // thread = (group of ranges, 4 consecutive d): it adds up the weighted partial sums of the ranges
    // g, g + GROUPS, ... once the first wave has worked out the weights; the groups are then added
    // in order through LDS. (Asking for the partial sums before the weights are known gains nothing:
    // a kernel this small takes 4.7 us whatever it does.)
    constexpr int CHUNKS = HD / 4;             // float4 chunks of a row
    constexpr int GROUPS = 256 / CHUNKS;       // 8 for HD = 128
    __shared__ float wgt[1024];
    __shared__ float sums[GROUPS][HD];
    __shared__ float s_inv;
    const int tid = threadIdx.x;
    const size_t bh = blockIdx.x;
    const int chunk = tid % CHUNKS, grp = tid / CHUNKS;
    // the first partial result of this sequence and head (with a list of ranges, see
    // attn_decode_kernel: [head, item], and the sequence has its own count of them)
    size_t first = bh * splits;
    if (ranges) {
        const int b = bh / nq, h = bh % nq;
        first = (size_t)h * splits + ranges[b];
        splits = ranges[b + 1] - ranges[b];
    }
    const float* ml = partial_ml + first * 2;

    if (tid < 64) {
        float M = -INFINITY;
        for (int s = tid; s < splits; s += 64) M = fmaxf(M, ml[2 * s]);
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) M = fmaxf(M, __shfl_xor(M, off, 64));
        float denom = 0.f;
        for (int s0 = 0; s0 < splits; s0 += 64) {
            const int s = s0 + tid;
            float w = 0.f, term = 0.f;
            if (s < splits && ml[2 * s] != -INFINITY) {
                w = fast_exp2((ml[2 * s] - M) * c);
                term = w * ml[2 * s + 1];
            }
            if (s < splits) wgt[s] = w;
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) term += __shfl_xor(term, off, 64);
            denom += term;
        }
        if (tid == 0) s_inv = denom > 0.f ? 1.0f / denom : 0.f;
    }
    __syncthreads();
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    if (grp < GROUPS)
        for (int s = grp; s < splits; s += GROUPS) {
            const f32x4 v = *(const f32x4*)(partial_o + (first + s) * HD + chunk * 4);
            acc += v * wgt[s];
        }
    if (grp < GROUPS) {
#pragma unroll
        for (int e = 0; e < 4; ++e) sums[grp][chunk * 4 + e] = acc[e];
    }
    __syncthreads();
    if (tid < HD) {
        float total = 0.f;
#pragma unroll
        for (int g = 0; g < GROUPS; ++g) total += sums[g][tid];
        out[bh * HD + tid] = hb_from_float<bf16>(total * s_inv);
    }
}

// ---------------------------------------------------------------- launchers
#define LOG2E 1.4426950408889634f

extern "C" int hb_attn_prefill_mfma(const void* q, const void* k_cache, const void* v_cache, void* out,
                                    const int* tile_seq, const int* tile_row0, const int* tile_rows,
                                    int num_tiles, const int* positions, const int* slots,
                                    const int* page_table, int max_pages, int page_size, int nq, int nkv,
                                    int hd, float scale, int window, int tile_height, hipStream_t stream) {
    HB_REQUIRE(num_tiles > 0 && nq > 0 && nkv > 0 && nq % nkv == 0, "attn_prefill: bad sizes");
    HB_REQUIRE(page_size == PAGE, "attn_prefill: pages must hold %d tokens", PAGE);
    HB_REQUIRE(window >= 0, "attn_prefill: bad window");
    HB_REQUIRE(scale > 0.f, "attn_prefill: the score scale must be positive");
    HB_REQUIRE(tile_height == 32 || tile_height == 64, "attn_prefill: tiles are 32 or 64 tokens high");
    const int G = nq / nkv;
    const int per_tile = nkv * ((G + 3) / 4);
    HB_REQUIRE((long)num_tiles * per_tile < (1l << 30), "attn_prefill: too many tiles");
    const int total = num_tiles * per_tile;
    const float c = scale * LOG2E;
    // tiles of 32 tokens: two groups of waves, each with two stages of keys and two of values;
    // tiles of 64: one ring of three stages of keys and three of values
    const size_t lds = (size_t)(tile_height == 64 ? 6 : 8) * PAGE * hd * sizeof(bf16);
#define LAUNCH_PREFILL(KERNEL, HDV)                                                                      \
    do {                                                                                                 \
        static bool allowed = false;            /* once a process (the attribute is the function's) */   \
        if (lds > 64 * 1024 && !allowed) {                                                               \
            hipError_t e_ = hipFuncSetAttribute((const void*)KERNEL<HDV>,                                \
                                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);   \
            HB_REQUIRE(e_ == hipSuccess, "attn_prefill: cannot have %zu bytes of LDS: %s", lds, hipGetErrorString(e_)); \
            allowed = true;                                                                              \
        }                                                                                                \
        KERNEL<HDV><<<total, 512, lds, stream>>>((const bf16*)q, (const bf16*)k_cache, (const bf16*)v_cache, \
                                                 (bf16*)out, tile_seq, tile_row0, tile_rows, positions, slots, \
                                                 page_table, max_pages, nq, nkv, c, window, per_tile);   \
    } while (0)
    if (tile_height == 64) {
        if (hd == 32) LAUNCH_PREFILL(attn_prefill_long_kernel, 32);
        else if (hd == 64) LAUNCH_PREFILL(attn_prefill_long_kernel, 64);
        else if (hd == 128) LAUNCH_PREFILL(attn_prefill_long_kernel, 128);
        else HB_REQUIRE(false, "attn_prefill: head_dim %d is not one of 32, 64, 128", hd);
    } else {
        if (hd == 32) LAUNCH_PREFILL(attn_prefill_kernel, 32);
        else if (hd == 64) LAUNCH_PREFILL(attn_prefill_kernel, 64);
        else if (hd == 128) LAUNCH_PREFILL(attn_prefill_kernel, 128);
        else HB_REQUIRE(false, "attn_prefill: head_dim %d is not one of 32, 64, 128", hd);
    }
#undef LAUNCH_PREFILL
    HB_CHECK_LAUNCH("attn_prefill");
    return 0;
}

// qkv != null: the fused form (see DecodeFusion); q is then not read. qkv_slices > 1 (2, 4 or 8, heads
// of 128 only): qkv is the first of that many slices of the projection's sums, slice_stride floats apart.
extern "C" int hb_attn_decode_mfma(const void* q, void* k_cache, void* v_cache, void* out,
                                   float* partial_o, float* partial_ml, const int* context_lens,
                                   const int* slots, const int* page_table, int max_pages, int page_size,
                                   int B, int nq, int nkv, int hd, float scale, int window, int splits,
                                   int pages_per_split, const float* qkv, const float* q_norm_w,
                                   const float* k_norm_w, const float* cos_t, const float* sin_t, float eps,
                                   int write_kv, int qkv_slices, size_t slice_stride, const int* ranges,
                                   hipStream_t stream) {
    // ranges != null: see attn_decode_kernel; `splits` is then the number of items of the grid (the
    // partial results are [nq, splits]), pages_per_split is not read
    HB_REQUIRE(!ranges || (B >= 2 && splits >= 2 && window == 0),
               "attn_decode: a list of ranges is for two sequences or more, with a merge, without a window");
    HB_REQUIRE(B > 0 && nq > 0 && nkv > 0 && nq % nkv == 0, "attn_decode: bad sizes");
    HB_REQUIRE(page_size == PAGE, "attn_decode: pages must hold %d tokens", PAGE);
    HB_REQUIRE(nq / nkv <= 32, "attn_decode: more than 32 query heads share a kv head");
    HB_REQUIRE(splits > 0 && splits <= 1024 && pages_per_split > 0 && nkv <= 65535, "attn_decode: bad split");
    HB_REQUIRE(window >= 0, "attn_decode: bad window");
    HB_REQUIRE(scale > 0.f, "attn_decode: the score scale must be positive");
    HB_REQUIRE(qkv_slices == 1 || (qkv && hd == 128 && (qkv_slices == 2 || qkv_slices == 4 || qkv_slices == 8) &&
                                   slice_stride >= (size_t)B * (nq + 2 * nkv) * hd),
               "attn_decode: %d slices of the projection are not taken here", qkv_slices);
    dim3 grid(ranges ? 1 : B, nkv, splits);
    const float c = scale * LOG2E;
    const DecodeFusion fu = {qkv, q_norm_w, k_norm_w, cos_t, sin_t, eps, write_kv, slice_stride};
    bf16* const direct = splits == 1 ? (bf16*)out : nullptr;      // one range: the kernel writes the output itself
    HB_REQUIRE(qkv || q, "attn_decode: neither q nor the projection rows are given");
    HB_REQUIRE((cos_t == nullptr) == (sin_t == nullptr), "attn_decode: cos and sin tables come together");
#define DECODE_ARGS(QPTR) QPTR, (bf16*)k_cache, (bf16*)v_cache, partial_o, partial_ml, context_lens, slots, \
                          page_table, max_pages, nq, nkv, c, window, pages_per_split, fu, direct, ranges, B
#define LAUNCH_DECODE(HDV) do {                                                                          \
    if (qkv)                                                                                             \
        attn_decode_kernel<HDV, true><<<grid, 64, 0, stream>>>(DECODE_ARGS(nullptr));                    \
    else                                                                                                 \
        attn_decode_kernel<HDV, false><<<grid, 64, 0, stream>>>(DECODE_ARGS((const bf16*)q));            \
    } while (0)
    if (qkv_slices == 2) attn_decode_kernel<128, true, 2><<<grid, 64, 0, stream>>>(DECODE_ARGS(nullptr));
    else if (qkv_slices == 4) attn_decode_kernel<128, true, 4><<<grid, 64, 0, stream>>>(DECODE_ARGS(nullptr));
    else if (qkv_slices == 8) attn_decode_kernel<128, true, 8><<<grid, 64, 0, stream>>>(DECODE_ARGS(nullptr));
    else
    if (hd == 32) LAUNCH_DECODE(32);
    else if (hd == 64) LAUNCH_DECODE(64);
    else if (hd == 128) LAUNCH_DECODE(128);
    else HB_REQUIRE(false, "attn_decode: head_dim %d is not one of 32, 64, 128", hd);
#undef LAUNCH_DECODE
#undef DECODE_ARGS
    HB_CHECK_LAUNCH("attn_decode");
    if (!direct) {
#define LAUNCH_MERGE(HDV) attn_decode_merge_kernel<HDV><<<B * nq, 256, 0, stream>>>(partial_o, partial_ml, (bf16*)out, splits, c, ranges, nq)
        if (hd == 32) LAUNCH_MERGE(32);
        else if (hd == 64) LAUNCH_MERGE(64);
        else LAUNCH_MERGE(128);
#undef LAUNCH_MERGE
        HB_CHECK_LAUNCH("attn_decode_merge");
    }
    return 0;
}
