"""Each kernel alone against a plain float32 formulation in torch, at sizes other than the
engine's: odd widths, heads and groups, sizes at and across tile edges."""
import math

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def dev():
    return torch.device("cuda", 0)


def rand(*shape, seed=0, scale=1.0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(dev())


# ---------------------------------------------------------------- plain kernels
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embed(dtype):
    from herbert_rs_amd.kernels import ops
    table = rand(37, 50, dtype=dtype)
    ids = torch.tensor([0, 36, 5, 5, 17], dtype=torch.int32, device=dev())
    out = torch.empty(5, 50, device=dev())
    ops.embed(ids, table, out)
    assert torch.equal(out, table[ids.long()].float())


@pytest.mark.parametrize("H", [64, 96, 1000, 4096, 5120])
def test_rmsnorm(H):
    from herbert_rs_amd.kernels import ops
    x = rand(7, H, seed=1, scale=3.0)
    w = 1 + 0.1 * rand(H, seed=2)
    for eps in (1e-6, 1e-5):
        want = x * torch.rsqrt((x.double() ** 2).mean(-1, keepdim=True) + eps).float() * w
        out = torch.empty_like(x)
        ops.rmsnorm(x, w, out, eps)
        assert torch.allclose(out, want, rtol=2e-6, atol=1e-6)
    rows = torch.tensor([6, 0, 3], dtype=torch.int32, device=dev())
    out = torch.empty(3, H, dtype=torch.bfloat16, device=dev())
    ops.rmsnorm(x, w, out, 1e-6, rows)
    want = (x[rows.long()] * torch.rsqrt((x[rows.long()] ** 2).mean(-1, keepdim=True) + 1e-6) * w)
    assert torch.allclose(out.float(), want, rtol=2 ** -8, atol=1e-6)


@pytest.mark.parametrize("M,N,K", [(1, 7, 5), (3, 65, 33), (64, 64, 16), (70, 130, 100), (129, 31, 257)])
@pytest.mark.parametrize("dts", [(torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16),
                                 (torch.float32, torch.bfloat16)])
def test_gemm_plain(M, N, K, dts):
    from herbert_rs_amd.kernels import ops
    a = rand(M, K, seed=3, dtype=dts[0])
    w = rand(N, K, seed=4, dtype=dts[1])
    want = (a.double() @ w.double().T).float()
    c = torch.empty(M, N, device=dev())
    ops.gemm_plain(a, w, c)
    assert torch.allclose(c, want, rtol=1e-5, atol=1e-5 * math.sqrt(K))
    base = rand(M, N, seed=5)
    c2 = base.clone()
    ops.gemm_plain(a, w, c2, accumulate=True)
    assert torch.allclose(c2, base + want, rtol=1e-5, atol=1e-5 * math.sqrt(K))
    cb = torch.empty(M, N, dtype=torch.bfloat16, device=dev())
    ops.gemm_plain(a, w, cb)
    assert torch.allclose(cb.float(), want, rtol=2 ** -8, atol=1e-3)


@pytest.mark.parametrize("I", [5, 128, 1000])
def test_swiglu(I):
    from herbert_rs_amd.kernels import ops
    gu = rand(6, 2 * I, seed=6, scale=4.0)
    gu[0, 0] = -90.0
    gu[0, 1] = 0.0
    want = torch.nn.functional.silu(gu[:, :I]) * gu[:, I:]
    out = torch.empty(6, I, device=dev())
    ops.swiglu(gu, out)
    assert torch.allclose(out, want, rtol=1e-5, atol=1e-6) and torch.isfinite(out).all()


# ------------------------------------------------------------------ MFMA GEMM
MFMA_SHAPES = [(1, 48, 32), (8, 4096, 4096), (16, 272, 96), (17, 1000, 224), (33, 96, 64), (48, 100, 128),
               (64, 24576, 512), (65, 128, 64), (128, 256, 128), (200, 330, 192), (2048, 512, 4096)]


@pytest.mark.parametrize("M,N,K", MFMA_SHAPES)
def test_gemm_mfma_store_and_add(M, N, K):
    from herbert_rs_amd.kernels import mfma
    a = rand(M, K, seed=7, dtype=torch.bfloat16)
    w = rand(N, K, seed=8, dtype=torch.bfloat16)
    assert mfma.gemm_supported(a, w)
    want = (a.double() @ w.double().T).float()
    c = torch.full((M, N), 7.0, device=dev())
    mfma.gemm(a, w, c)
    tol = 2e-6 * K ** 0.5 * float(want.abs().max()) + 1e-4      # float32 accumulation of exact products
    assert float((c - want).abs().max()) <= tol
    base = rand(M, N, seed=9)
    c2 = base.clone()
    mfma.gemm(a, w, c2, accumulate=True)
    assert float((c2 - (base + want)).abs().max()) <= tol


@pytest.mark.parametrize("tile", [188, 142, 122, 2188, 4142])
@pytest.mark.parametrize("M,N,K", [(300, 520, 1024), (257, 1028, 1024), (640, 330, 1024), (129, 257, 1024)])
def test_gemm_mfma_large_tiles_with_ragged_edges(M, N, K, tile):
    """The large tiles by name, whole and with K cut, for sizes that end inside a tile: their
    float32 outputs leave through LDS a row at a time where N is a multiple of 4, lane by lane
    otherwise, and rows and columns past the end are never written."""
    from herbert_rs_amd.kernels import mfma
    a = rand(M, K, seed=17, dtype=torch.bfloat16)
    w = rand(N, K, seed=18, dtype=torch.bfloat16)
    want = (a.double() @ w.double().T).float()
    tol = 2e-6 * K ** 0.5 * float(want.abs().max()) + 1e-4
    for packed in (False, True):
        if packed and N % 16:
            continue
        wt = mfma.pack_weight(w) if packed else w
        c = torch.full((M + 1, N), 7.0, device=dev())          # a row behind the last one
        mfma.gemm(a, wt, c[:M], packed=packed, tile=tile)
        assert float((c[:M] - want).abs().max()) <= tol
        assert float((c[M] - 7.0).abs().max()) == 0.0
        base = rand(M, N, seed=19)
        c2 = base.clone()
        mfma.gemm(a, wt, c2, accumulate=True, packed=packed, tile=tile)
        assert float((c2 - (base + want)).abs().max()) <= tol


@pytest.mark.parametrize("M,I,K", [(1, 16, 32), (8, 12288, 4096), (40, 48, 96), (64, 1024, 64),
                                   (100, 176, 128), (300, 256, 64)])
def test_gemm_mfma_swiglu(M, I, K):
    from herbert_rs_amd.kernels import mfma
    a = rand(M, K, seed=10, dtype=torch.bfloat16, scale=0.5)
    gate = rand(I, K, seed=11, dtype=torch.bfloat16, scale=0.3)
    up = rand(I, K, seed=12, dtype=torch.bfloat16, scale=0.3)
    w = mfma.interleave_gate_up(gate, up)
    g = a.double() @ gate.double().T
    u = a.double() @ up.double().T
    want = (g / (1 + torch.exp(-g)) * u).float()
    out = torch.empty(M, I, dtype=torch.bfloat16, device=dev())
    mfma.gemm_swiglu(a, w, out)
    err = (out.float() - want).abs()
    assert float((err - 2 ** -8 * want.abs()).max()) <= 1e-3 * float(want.abs().max()) + 1e-5


@pytest.mark.parametrize("M,I,K,tile", [(300, 256, 128, 168), (257, 1040, 1024, 168), (512, 96, 64, 168), (70, 304, 256, 168),
                                        (1024, 1536, 512, 168), (64, 480, 256, 164), (33, 1040, 1024, 164), (50, 96, 64, 164),
                                        (130, 304, 128, 164)])
def test_gemm_mfma_swiglu_tiles_with_three_pieces_a_wave(M, I, K, tile):
    """The SwiGLU product on tiles whose waves hold three pieces of 32 columns (192 columns by
    four waves, 96 by two), by name: sizes that end inside a tile in both directions, weights as
    stored and packed; rows past the end are not written."""
    from herbert_rs_amd.kernels import mfma
    a = rand(M, K, seed=20, dtype=torch.bfloat16, scale=0.5)
    gate = rand(I, K, seed=21, dtype=torch.bfloat16, scale=0.3)
    up = rand(I, K, seed=22, dtype=torch.bfloat16, scale=0.3)
    w = mfma.interleave_gate_up(gate, up)
    g = a.double() @ gate.double().T
    u = a.double() @ up.double().T
    want = (g / (1 + torch.exp(-g)) * u).float()
    for packed in (False, True):
        out = torch.full((M + 1, I), 3.0, dtype=torch.bfloat16, device=dev())
        mfma.gemm_swiglu(a, mfma.pack_weight(w) if packed else w, out[:M], packed, tile=tile)
        err = (out[:M].float() - want).abs()
        assert float((err - 2 ** -8 * want.abs()).max()) <= 1e-3 * float(want.abs().max()) + 1e-5
        assert float((out[M].float() - 3.0).abs().max()) == 0.0
    c = torch.zeros(M, 2 * I, device=dev())
    with pytest.raises(Exception, match="SwiGLU product whole only"):
        mfma.gemm(a, w, c, tile=tile)


@pytest.mark.parametrize("M,N,K,cut", [(300, 256, 128, -128), (257, 96, 64, -256), (530, 512, 256, -256), (129, 64, 64, -128),
                                       (2049, 512, 128, 0), (2060, 4096, 4096, 0)])
def test_gemm_mfma_rows_cut_into_two_products(M, N, K, cut):
    """A product cut in two along its rows (whole tiles, then the rest, each a product of its own;
    by name, and at the last sizes by the kernel's own estimates, which cut the 8B shape's products
    of 2,060 rows at 2,048): store, add and SwiGLU give what the product whole gives, and nothing
    beyond the rows is written."""
    from herbert_rs_amd.kernels import mfma
    if (M, N, K) == (2060, 4096, 4096):
        assert mfma.gemm_split(M, N, K, mfma.EPI_ADD) == 2048 and mfma.gemm_split(M, N, K, mfma.EPI_STORE) == 2048
    a = rand(M, K, seed=30, dtype=torch.bfloat16, scale=0.5)
    w = rand(N, K, seed=31, dtype=torch.bfloat16, scale=0.3)
    want = a.double() @ w.double().T
    wp = mfma.pack_weight(w)
    out = torch.full((M + 1, N), 3.0, device=dev())
    mfma.gemm(a, wp, out[:M], False, True, tile=cut)
    assert float((out[:M].double() - want).abs().max()) <= 1e-5 * float(want.abs().max()) + 1e-6
    assert float((out[M] - 3.0).abs().max()) == 0.0
    mfma.gemm(a, wp, out[:M], True, True, tile=cut)
    assert float((out[:M].double() - 2 * want).abs().max()) <= 2e-5 * float(want.abs().max()) + 1e-6
    gate, up = w[:N // 2], w[N // 2:]
    g, u = a.double() @ gate.double().T, a.double() @ up.double().T
    act = (g / (1 + torch.exp(-g)) * u).float()
    half = torch.full((M + 1, N // 2), 3.0, dtype=torch.bfloat16, device=dev())
    mfma.gemm_swiglu(a, mfma.pack_weight(mfma.interleave_gate_up(gate, up)), half[:M], True, tile=cut)
    err = (half[:M].float() - act).abs()
    assert float((err - 2 ** -8 * act.abs()).max()) <= 1e-3 * float(act.abs().max()) + 1e-5
    assert float((half[M].float() - 3.0).abs().max()) == 0.0


def test_gemm_mfma_refuses_what_it_cannot_do():
    from herbert_rs_amd.kernels import mfma
    a = rand(4, 40, dtype=torch.bfloat16)
    w = rand(8, 40, dtype=torch.bfloat16)
    assert not mfma.gemm_supported(a, w)
    assert not mfma.gemm_supported(a.float(), w)


# ------------------------------------------------------------------ attention
class FakeMeta:
    pass


def paged_case(lengths, new_counts, nkv, hd, dtype, seed=0, n_pages=64, shuffle=True):
    """A cache filled with random keys and values for sequences of the given lengths, the last
    new_counts[i] positions of each being the step's tokens. Returns (meta, kv, K, V) with K, V
    the dense per-sequence tensors [len, nkv, hd]."""
    from herbert_rs_amd.cache.paged import LayerKV
    g = torch.Generator().manual_seed(seed)
    pages_per_slot = max(16, (max(lengths) + 63) // 64)
    B = len(lengths)
    table = torch.zeros(B + 2, pages_per_slot, dtype=torch.int32)
    order = torch.randperm(n_pages, generator=g).tolist() if shuffle else list(range(n_pages))
    k_pool = torch.zeros(n_pages, nkv, 64, hd)
    v_pool = torch.zeros(n_pages, nkv, hd, 64)
    dense = []
    slots = [b + 1 for b in range(B)]          # slot ids differ from batch indices
    for b, n in enumerate(lengths):
        K = torch.randn(n, nkv, hd, generator=g).to(dtype).float()
        V = torch.randn(n, nkv, hd, generator=g).to(dtype).float()
        dense.append((K, V))
        for p in range((n + 63) // 64):
            page = order.pop()
            table[slots[b], p] = page
            chunk = slice(p * 64, min(n, (p + 1) * 64))
            cnt = chunk.stop - chunk.start
            k_pool[page, :, :cnt] = K[chunk].transpose(0, 1)
            v_pool[page, :, :, :cnt] = V[chunk].permute(1, 2, 0)
    kv = LayerKV(k_pool.to(dtype).to(dev()), v_pool.to(dtype).to(dev()), table.to(dev()), 64, 0)
    meta = FakeMeta()
    pos, seq = [], []
    starts = [0]
    for b, (n, c) in enumerate(zip(lengths, new_counts)):
        pos += list(range(n - c, n))
        seq += [b] * c
        starts.append(starts[-1] + c)
    meta.positions = torch.tensor(pos, dtype=torch.int32, device=dev())
    meta.seq_of = torch.tensor(seq, dtype=torch.int32, device=dev())
    meta.slots = torch.tensor(slots, dtype=torch.int32, device=dev())
    meta.context_lens = torch.tensor(lengths, dtype=torch.int32, device=dev())
    meta.num_seqs, meta.num_tokens = B, len(pos)
    meta.max_new, meta.max_context, meta.max_position = max(new_counts), max(lengths), max(lengths) - 1
    import numpy as np
    meta.host_starts = np.array(starts, dtype=np.int32)
    meta.host_context = np.array(lengths, dtype=np.int32)
    meta.derived = {}
    from herbert_rs_amd.engine.batch import BatchMeta, bucket, unequal_level
    meta.context_bucket = bucket(max(lengths))
    # contexts of very unequal lengths: the decode kernel deals its grid out by a list of ranges
    meta.unequal, meta.static, meta.token_ids = unequal_level(lengths), None, meta.positions
    meta.ranges_for = lambda items, unit: BatchMeta.ranges_for(meta, items, unit)
    return meta, kv, dense


def attention_reference(q, meta, dense, nq, nkv, hd, scale, window):
    out = torch.zeros(q.shape[0], nq, hd)
    qf = q.float().cpu().view(-1, nq, hd)
    pos = meta.positions.cpu().tolist()
    seq = meta.seq_of.cpu().tolist()
    for t in range(q.shape[0]):
        K, V = dense[seq[t]]
        lo = max(0, pos[t] + 1 - window) if window else 0
        for h in range(nq):
            g = h // (nq // nkv)
            s = (K[lo:pos[t] + 1, g] @ qf[t, h]) * scale
            p = torch.softmax(s.double(), 0).float()
            out[t, h] = (p[:, None] * V[lo:pos[t] + 1, g]).sum(0)
    return out.view(q.shape[0], nq * hd)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nq,nkv,hd,window", [(4, 2, 16, 0), (6, 2, 32, 0), (5, 1, 48, 70), (3, 3, 80, 0),
                                              (2, 1, 256, 130)])
def test_attention_plain(nq, nkv, hd, window, dtype):
    from herbert_rs_amd.kernels import ops
    lengths, new = [5, 200, 64, 129], [5, 70, 1, 129]
    meta, kv, dense = paged_case(lengths, new, nkv, hd, dtype, seed=nq)
    q = rand(sum(new), nq * hd, seed=20, dtype=dtype)
    out = torch.empty_like(q)
    scale = hd ** -0.5
    ops.attention_plain(q, meta, kv, out, nq, nkv, hd, scale, window)
    want = attention_reference(q, meta, dense, nq, nkv, hd, scale, window)
    tol = 2e-5 if dtype == torch.float32 else 2 ** -7
    assert float((out.float().cpu() - want).abs().max()) <= tol * float(want.abs().max())


@pytest.mark.parametrize("tile_height", [32, 64])
@pytest.mark.parametrize("nq,nkv,hd,window", [(4, 1, 128, 0), (8, 2, 64, 0), (6, 2, 32, 0), (5, 1, 64, 70),
                                              (3, 3, 128, 100), (16, 2, 128, 0), (2, 2, 32, 0)])
def test_attention_mfma_prefill(nq, nkv, hd, window, tile_height):
    """Both prompt kernels, each asked for by name: tiles of 32 tokens (two groups of waves take a
    tile's pages in turn) and tiles of 64 (two halves share the pages). Sequences that start in
    the cache at positions that no tile height divides, tiles of 1 to 64 rows, windows."""
    from herbert_rs_amd.kernels import mfma
    lengths, new = [5, 200, 64, 129, 33, 300, 450], [5, 70, 2, 129, 32, 300, 97]
    meta, kv, dense = paged_case(lengths, new, nkv, hd, torch.bfloat16, seed=nq + hd)
    q = rand(sum(new), nq * hd, seed=21, dtype=torch.bfloat16)
    out = torch.full_like(q, 9.0)
    scale = hd ** -0.5
    assert mfma.attention_supported(q, kv, nq, nkv, hd)
    mfma.attention(q, meta, kv, out, nq, nkv, hd, scale, window, tile_height=tile_height)
    want = attention_reference(q, meta, dense, nq, nkv, hd, scale, window)
    # probabilities and the output are rounded to bfloat16 (2^-9 each)
    assert float((out.float().cpu() - want).abs().max()) <= 2 ** -7 * float(want.abs().max())


@pytest.mark.parametrize("nq,nkv,hd,window", [(4, 1, 128, 0), (32, 8, 128, 0), (6, 2, 32, 0), (5, 1, 64, 70),
                                              (3, 3, 128, 100), (64, 2, 64, 0)])
@pytest.mark.parametrize("lengths", [[1, 64, 65, 700], [1000], [130, 3, 512, 999, 77, 640, 64, 128, 256]])
@pytest.mark.parametrize("waves,by_list", [(1024, True), (1024, False), (1, False)])
def test_attention_mfma_decode(nq, nkv, hd, window, lengths, waves, by_list, monkeypatch):
    """waves = 1: every sequence is one range, and the kernel writes the output without a merge.
    by_list: where the lengths are very unequal (and there is no window) the grid is dealt out by a
    list of ranges; without it every sequence has the same number of ranges."""
    from herbert_rs_amd.kernels import mfma
    monkeypatch.setattr(mfma, "DECODE_WAVES", waves)
    meta, kv, dense = paged_case(lengths, [1] * len(lengths), nkv, hd, torch.bfloat16, seed=nq + hd,
                                 n_pages=80)
    meta.unequal = meta.unequal and by_list
    assert (mfma._decode_ranges(meta, nkv, window) is not None) == (by_list and len(lengths) > 1 and not window)
    q = rand(len(lengths), nq * hd, seed=22, dtype=torch.bfloat16)
    out = torch.full_like(q, 9.0)
    scale = hd ** -0.5
    mfma.attention(q, meta, kv, out, nq, nkv, hd, scale, window)
    want = attention_reference(q, meta, dense, nq, nkv, hd, scale, window)
    assert float((out.float().cpu() - want).abs().max()) <= 2 ** -7 * float(want.abs().max())


@pytest.mark.parametrize("lengths", [[20000, 70, 1000, 64, 1, 65, 130, 900], [300] * 30 + [9000, 5000],
                                     [64] * 63 + [4000], [8000, 1, 1], [64] * 129 + [6000]])
def test_attention_mfma_decode_of_unequal_sequences_by_a_list(lengths):
    """Sequences of very unequal lengths: the grid's items are dealt out by a list, every item a
    range of the same number of pages of whichever sequence. In each sequence one key far back (in
    its first page, at a page's edge, in its last range) scores far above the rest, so that a range
    that is skipped, read twice or given to another sequence shows."""
    from herbert_rs_amd.engine.batch import range_list
    from herbert_rs_amd.kernels import mfma
    nq, nkv, hd = 16, 8, 128
    B = len(lengths)
    pages = sum((n + 64) // 64 + 1 for n in lengths)
    meta, kv, dense = paged_case(lengths, [1] * B, nkv, hd, torch.bfloat16, seed=B, n_pages=pages)
    items, listed = mfma._decode_ranges(meta, nkv, 0)
    assert items == max(128, 2 * B)
    got = listed.cpu().numpy()
    assert (got == range_list(lengths, items, 64)).all() and got[B] <= items
    per = int(got[B + 1])
    assert all((got[b + 1] - got[b]) * per >= -(-n // 64) > (got[b + 1] - got[b] - 1) * per for b, n in enumerate(lengths))
    targets = [[0, 63, 64, n - 2, (n - 1) // 64 * 64, n // 2][b % 6] % max(1, n - 1) for b, n in enumerate(lengths)]
    q = torch.zeros(B, nq * hd)
    for b, t in enumerate(targets):
        q[b] = (dense[b][0][t] * 8).repeat_interleave(nq // nkv, dim=0).reshape(-1)    # each head with its kv head's key
    q = q.to(torch.bfloat16).to(dev())
    out = torch.full_like(q, 9.0)
    mfma.attention(q, meta, kv, out, nq, nkv, hd, 1.0, 0)
    want = attention_reference(q, meta, dense, nq, nkv, hd, 1.0, 0)
    assert float((out.float().cpu() - want).abs().max()) <= 2 ** -7 * float(want.abs().max())
    res = out.float().cpu().view(B, nq, hd)
    for b, t in enumerate(targets):
        if lengths[b] > 1:
            V = dense[b][1][t].repeat_interleave(nq // nkv, dim=0)
            assert float((res[b] - V).abs().max()) < 0.05, (b, t)


def test_attention_mfma_decode_of_many_sequences_in_shorter_ranges():
    """70 sequences on 8 kv heads are 560 waves of one range each: three on some CUs where most have
    two. The host then cuts every context into shorter ranges (here six) with a merge, as it does
    for few sequences; with 64 sequences, which sit evenly, every sequence stays one range."""
    from herbert_rs_amd.kernels import mfma
    nq, nkv, hd = 16, 8, 128
    lengths = [1100 + (37 * i) % 230 for i in range(70)]
    meta, kv, dense = paged_case(lengths, [1] * len(lengths), nkv, hd, torch.bfloat16, seed=5, n_pages=70 * 21 + 8)
    assert mfma._decode_split(meta, nkv, 0)[0] == 6
    q = rand(len(lengths), nq * hd, seed=26, dtype=torch.bfloat16)
    out = torch.full_like(q, 9.0)
    mfma.attention(q, meta, kv, out, nq, nkv, hd, hd ** -0.5, 0)
    want = attention_reference(q, meta, dense, nq, nkv, hd, hd ** -0.5, 0)
    assert float((out.float().cpu() - want).abs().max()) <= 2 ** -7 * float(want.abs().max())
    meta64, _, _ = paged_case(lengths[:64], [1] * 64, nkv, hd, torch.bfloat16, seed=5, n_pages=64 * 21 + 8)
    assert mfma._decode_split(meta64, nkv, 0)[0] == 1


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nq,nkv,hd,rot,norm", [(4, 2, 128, 128, True), (3, 1, 64, 64, False), (2, 2, 96, 0, True),
                                                (5, 1, 32, 32, True), (2, 1, 80, 40, True), (1, 1, 256, 256, True),
                                                (6, 2, 48, 48, True), (2, 1, 112, 112, True), (3, 1, 16, 16, True)])
def test_qk_norm_rope_write(nq, nkv, hd, rot, norm, dtype):
    """Per-head norm, rotation and the write into the pages, for prompts that cross pages and a
    step that is no multiple of 64 tokens (the tiled kernel), and for a few tokens (the plain one)."""
    from herbert_rs_amd.kernels import ops
    for lengths, new in (([130, 70, 300, 64], [130, 7, 190, 64]), ([5, 90], [2, 1])):
        meta, kv, _ = paged_case(lengths, new, nkv, hd, dtype, seed=hd)
        before_k, before_v = kv.k.clone(), kv.v.clone()
        T = sum(new)
        qkv = rand(T, (nq + 2 * nkv) * hd, seed=50, scale=1.3)
        qw = (1 + rand(hd, seed=51, scale=0.3)) if norm else None
        kw = (1 + rand(hd, seed=52, scale=0.3)) if norm else None
        cos = sin = None
        if rot:
            ang = torch.arange(512, dtype=torch.float32)[:, None] * (10000.0 ** (-torch.arange(rot // 2) / (rot // 2)))[None]
            cos, sin = ang.cos().to(dev()).contiguous(), ang.sin().to(dev()).contiguous()
        eps = 1e-5
        q = torch.full((T, nq * hd), 9.0, dtype=dtype, device=dev())
        ops.qk_norm_rope_write(qkv, qw, kw, cos, sin, rot, meta, kv, q, nq, nkv, hd, eps)
        if ops.rope_write_adds_slices(T, hd, rot, dtype, True, cos is not None):
            # the same rows in 2, 4 or 8 slices that sum to them exactly: the kernel adds them up
            from herbert_rs_amd.cache.paged import LayerKV
            for n in ops.ROPE_WRITE_SLICES:
                parts = torch.zeros(n, *qkv.shape, device=dev())
                coarse = (qkv * 8).round() / 8
                parts[0], parts[n - 1] = coarse / 2, coarse / 2
                parts[n // 2] += qkv - coarse
                assert torch.equal(parts.sum(0), qkv)
                kv_s = LayerKV(before_k.clone(), before_v.clone(), kv.page_table, kv.page_size, 0)
                q_s = torch.full_like(q, 5.0)
                ops.qk_norm_rope_write(torch.empty_like(qkv), qw, kw, cos, sin, rot, meta, kv_s, q_s, nq, nkv, hd, eps,
                                       qkv_slices=(n, parts.data_ptr(), qkv.numel()))
                assert torch.equal(q_s, q) and torch.equal(kv_s.k, kv.k) and torch.equal(kv_s.v, kv.v), n

        x = qkv.double().cpu().view(T, nq + 2 * nkv, hd)
        pos = meta.positions.cpu().long()

        def head_op(v, w):
            if w is not None:
                v = v / torch.sqrt((v ** 2).mean(-1, keepdim=True) + eps) * w.double().cpu()
            if rot:
                c, s_ = cos.double().cpu()[pos][:, None, :], sin.double().cpu()[pos][:, None, :]
                a, b = v[..., :rot // 2], v[..., rot // 2:rot]
                v = torch.cat([a * c - b * s_, a * s_ + b * c, v[..., rot:]], -1)
            return v
        want_q = head_op(x[:, :nq], qw).reshape(T, nq * hd)
        want_k = head_op(x[:, nq:nq + nkv], kw)
        want_v = x[:, nq + nkv:]
        tol = 1e-5 if dtype == torch.float32 else 2 ** -8
        assert float((q.double().cpu() - want_q).abs().max()) <= tol * float(want_q.abs().max())
        table = kv.page_table.cpu()
        slots, seq = meta.slots.cpu().tolist(), meta.seq_of.cpu().tolist()
        exp_k, exp_v = before_k.double().cpu(), before_v.double().cpu()
        for t in range(T):
            p = int(pos[t])
            page = int(table[slots[seq[t]], p // 64])
            exp_k[page, :, p % 64] = want_k[t]
            exp_v[page, :, :, p % 64] = want_v[t]
        # every other place of the pages is as it was
        assert float((kv.k.double().cpu() - exp_k).abs().max()) <= tol * float(exp_k.abs().max())
        assert float((kv.v.double().cpu() - exp_v).abs().max()) <= tol * float(exp_v.abs().max())


@pytest.mark.parametrize("shape", [0, 1, 2])
@pytest.mark.parametrize("packed", [True, False])
@pytest.mark.parametrize("nq,nkv,norm,rope", [(4, 2, True, True), (3, 1, False, True), (2, 2, True, False), (1, 1, True, True)])
def test_gemm_qkv_with_norm_rotation_and_cache_write(nq, nkv, norm, rope, packed, shape):
    """The q/k/v projection that norms, rotates and writes the pages in its epilogue against the
    product followed by the kernel of its own: prompts that cross pages, rows that are no
    multiple of the tile, an odd number of heads (half a tile of columns is empty)."""
    from herbert_rs_amd.cache.paged import LayerKV
    from herbert_rs_amd.kernels import mfma, ops
    hd, K = 128, 192
    lengths, new = [330, 70, 300, 64], [330, 7, 190, 64]
    meta, kv, _ = paged_case(lengths, new, nkv, hd, torch.bfloat16, seed=nq)
    kv2 = LayerKV(kv.k.clone(), kv.v.clone(), kv.page_table, 64, 0)
    T = sum(new)
    a = rand(T, K, seed=70, dtype=torch.bfloat16)
    w = rand((nq + 2 * nkv) * hd, K, seed=71, dtype=torch.bfloat16, scale=0.1)
    qw = (1 + rand(hd, seed=72, scale=0.3)) if norm else None
    kw = (1 + rand(hd, seed=73, scale=0.3)) if norm else None
    cos = sin = None
    if rope:
        ang = torch.arange(512, dtype=torch.float32)[:, None] * (10000.0 ** (-torch.arange(hd // 2) / (hd // 2)))[None]
        cos, sin = ang.cos().to(dev()).contiguous(), ang.sin().to(dev()).contiguous()
    eps = 1e-5
    wp = mfma.pack_weight(w) if packed else w
    qkv = torch.empty(T, (nq + 2 * nkv) * hd, device=dev())
    mfma.gemm(a, wp, qkv, packed=packed)
    want_q = torch.full((T, nq * hd), 9.0, dtype=torch.bfloat16, device=dev())
    ops.qk_norm_rope_write(qkv, qw, kw, cos, sin, hd if rope else 0, meta, kv, want_q, nq, nkv, hd, eps)
    got_q = torch.full((T, nq * hd), 7.0, dtype=torch.bfloat16, device=dev())
    old = mfma.QKV_FUSE_MIN_TILES
    mfma.QKV_FUSE_MIN_TILES = 1          # (the engine takes this path only when its tiles fill the GPU)
    try:
        assert mfma.gemm_qkv_fusable(a, wp, meta, kv2, nq, nkv, hd, hd if rope else 0)
    finally:
        mfma.QKV_FUSE_MIN_TILES = old
    mfma.gemm_qkv(a, wp, packed, qw, kw, cos, sin, meta, kv2, got_q, nq, nkv, hd, eps, shape=shape)
    # the two paths add the squares and the products in other orders: an element may round the other way
    for got, want in ((got_q, want_q), (kv2.k, kv.k), (kv2.v, kv.v)):
        d = (got.float() - want.float()).abs()
        assert float(d.max()) <= 2 ** -7 * float(want.float().abs().max())
        assert float((d > 0).float().mean()) < 2e-2


@pytest.mark.parametrize("nq,nkv,hd,window,norm,rope", [(4, 1, 128, 0, True, True), (32, 8, 128, 0, True, True),
                                                        (6, 2, 32, 0, True, False), (5, 1, 64, 70, False, True),
                                                        (3, 3, 128, 100, True, True), (64, 2, 64, 0, False, False)])
@pytest.mark.parametrize("lengths", [[1, 64, 65, 700], [1000], [130, 3, 512, 999, 77, 640, 64, 128, 256]])
@pytest.mark.parametrize("waves,by_list", [(1024, True), (1024, False), (1, False)])
def test_attention_mfma_decode_fused_with_norm_rotation_and_cache_write(nq, nkv, hd, window, norm, rope, lengths,
                                                                        waves, by_list, monkeypatch):
    """The decode kernel that norms, rotates and writes the new key and value itself against the
    separate kernels: same pages afterwards, same output (waves = 1: without a merge; by_list: very
    unequal lengths by a list of ranges, in both kernels)."""
    from herbert_rs_amd.cache.paged import LayerKV
    from herbert_rs_amd.kernels import mfma, ops
    monkeypatch.setattr(mfma, "DECODE_WAVES", waves)
    B = len(lengths)
    meta, kv, _ = paged_case(lengths, [1] * B, nkv, hd, torch.bfloat16, seed=nq + hd, n_pages=80)
    meta.unequal = meta.unequal and by_list
    kv2 = LayerKV(kv.k.clone(), kv.v.clone(), kv.page_table, 64, 0)
    before_k, before_v = kv.k.clone(), kv.v.clone()
    qkv = rand(B, (nq + 2 * nkv) * hd, seed=23, scale=1.5)
    qw = (1 + rand(hd, seed=24, scale=0.3)) if norm else None
    kw = (1 + rand(hd, seed=25, scale=0.3)) if norm else None
    cos = sin = None
    if rope:
        ang = torch.arange(1024, dtype=torch.float32)[:, None] * (10000.0 ** (-torch.arange(hd // 2) / (hd // 2)))[None]
        cos, sin = ang.cos().to(dev()).contiguous(), ang.sin().to(dev()).contiguous()
    scale, eps = hd ** -0.5, 1e-5
    assert mfma.decode_fusable(meta, kv, nq, nkv, hd, hd if rope else 0, torch.bfloat16)
    q = torch.empty(B, nq * hd, dtype=torch.bfloat16, device=dev())
    want = torch.full_like(q, 9.0)
    ops.qk_norm_rope_write(qkv, qw, kw, cos, sin, hd if rope else 0, meta, kv, q, nq, nkv, hd, eps)
    mfma.attention(q, meta, kv, want, nq, nkv, hd, scale, window)
    got = torch.full_like(q, 7.0)
    mfma.attention_decode_fused(qkv, qw, kw, cos, sin, meta, kv2, got, nq, nkv, hd, eps, scale, window)
    if hd == 128:
        # the same projection rows in 2, 4 or 8 slices that sum to them exactly: the kernel adds them up
        for n in mfma.DEFERRED_SLICES:
            parts = torch.zeros(n, *qkv.shape, device=dev())
            coarse = (qkv * 8).round() / 8                  # leaves a remainder that float32 adds back exactly
            parts[0], parts[n - 1] = coarse / 2, coarse / 2
            parts[n // 2] += qkv - coarse
            assert torch.equal(parts.sum(0), qkv)
            kv3 = LayerKV(kv2.k.clone().fill_(0), kv2.v.clone().fill_(0), kv.page_table, 64, 0)
            kv3.k.copy_(before_k), kv3.v.copy_(before_v)
            sliced = torch.full_like(q, 5.0)
            mfma.attention_decode_fused(torch.empty_like(qkv), qw, kw, cos, sin, meta, kv3, sliced, nq, nkv, hd, eps,
                                        scale, window, qkv_slices=(n, parts.data_ptr(), qkv.numel()))
            assert torch.equal(sliced, got) and torch.equal(kv3.k, kv2.k) and torch.equal(kv3.v, kv2.v), n
    assert torch.equal(kv.v, kv2.v)
    # the two kernels sum the squares in another order: a key element may round the other way
    dk = (kv.k.float() - kv2.k.float()).abs()
    assert float(dk.max()) <= 2 ** -7 * float(kv.k.float().abs().max())
    assert float((dk > 0).float().mean()) < 1e-3
    w = want.float()
    assert float((got.float() - w).abs().max()) <= 2 ** -6 * float(w.abs().max())


def test_attention_finds_one_far_key_among_hundreds():
    """One key far back scores far above the rest: the output must be its value, whichever page
    and split it lies in. Random keys would hide a page or a split that is skipped."""
    from herbert_rs_amd.kernels import mfma, ops
    nq, nkv, hd = 4, 1, 64
    for n, target in ((900, 3), (900, 64 * 7 + 63), (900, 899), (257, 192), (20000, 11), (20000, 64 * 200 + 5)):
        for mode in ("decode", "prefill"):
            new = 1 if mode == "decode" else 40
            meta, kv, dense = paged_case([n], [new], nkv, hd, torch.bfloat16, seed=target, n_pages=max(64, n // 64 + 2))
            K, V = dense[0]
            q = torch.zeros(new, nq * hd)
            q[:, :] = (K[target, 0] * 8).repeat(nq)          # aligned with that key, scaled up
            q = q.to(torch.bfloat16).to(dev())
            if target >= n - new:
                continue
            for fn in (mfma.attention, ops.attention_plain):
                out = torch.empty_like(q)
                fn(q, meta, kv, out, nq, nkv, hd, 1.0, 0)
                got = out.float().cpu().view(new, nq, hd)
                assert float((got - V[target, 0]).abs().max()) < 0.02, (n, target, mode, fn.__name__)


@pytest.mark.parametrize("M,N,K", [(1, 48, 32), (8, 4096, 4096), (17, 1008, 224), (64, 24576, 512),
                                   (65, 128, 64), (200, 336, 192), (2048, 512, 4096)])
def test_gemm_mfma_packed_weights(M, N, K):
    from herbert_rs_amd.kernels import mfma
    a = rand(M, K, seed=7, dtype=torch.bfloat16)
    w = rand(N, K, seed=8, dtype=torch.bfloat16)
    plain = torch.empty(M, N, device=dev())
    mfma.gemm(a, w, plain)
    packed = torch.empty(M, N, device=dev())
    mfma.gemm(a, mfma.pack_weight(w), packed, packed=True)
    assert torch.equal(plain, packed)


@pytest.mark.parametrize("M,N,K,packed", [(1, 16384, 32, False), (8, 24576, 4096, True), (16, 16400, 96, False),
                                          (3, 17024, 64, True)])
def test_gemm_mfma_with_fused_norm(M, N, K, packed):
    from herbert_rs_amd.kernels import mfma
    x = rand(M, K, seed=30, scale=2.0)
    g = 1 + 0.1 * rand(K, seed=31)
    w = rand(N, K, seed=32, dtype=torch.bfloat16, scale=0.1)
    eps = 1e-6
    inv = torch.rsqrt((x.double() ** 2).mean(-1, keepdim=True) + eps)
    # the kernel rounds x * g to bfloat16 and applies inv to the float32 sums
    xg = (x * g).to(torch.bfloat16).double()
    want = ((xg @ w.double().T) * inv).float()
    out = torch.empty(M, N, device=dev())
    mfma.gemm(x, mfma.pack_weight(w) if packed else w, out, packed=packed, norm=(g, eps))
    assert float((out - want).abs().max()) <= 1e-5 * float(want.abs().max()) + 1e-5
    exact = ((x.double() * inv * g) @ w.double().T).float()          # and near the unrounded norm
    assert float((out - exact).abs().max()) <= 2 ** -7 * float(exact.abs().max())
    if N % 32 == 0:
        gate, up = w[:N // 2].contiguous(), w[N // 2:].contiguous()
        wi = mfma.interleave_gate_up(gate, up)
        act = torch.empty(M, N // 2, dtype=torch.bfloat16, device=dev())
        mfma.gemm_swiglu(x, mfma.pack_weight(wi) if packed else wi, act, packed=packed, norm=(g, eps))
        gg, uu = (xg @ gate.double().T) * inv, (xg @ up.double().T) * inv
        wanted = (gg / (1 + torch.exp(-gg)) * uu).float()
        assert float((act.float() - wanted).abs().max()) <= 2 ** -7 * float(wanted.abs().max()) + 1e-5


@pytest.mark.parametrize("M,H,K1,N2,packed", [(1, 64, 32, 48, False), (8, 4096, 1024, 6144, True), (16, 1056, 96, 16448, False),
                                              (5, 2336, 160, 2304, True), (13, 17024, 64, 64, True),
                                              (7, 1048, 64, 0, False), (8, 4096, 64, 24576, True),
                                              (11, 1088, 96, 16512, False), (1, 576, 32, 16384, True),
                                              (8, 5120, 8192, 6144, True), (3, 5124, 16384, 0, False)])
def test_gemm_mfma_hands_a_norm_to_the_next_product(M, H, K1, N2, packed):
    """x += a W1^T leaves bf16(x g) and the squares of x by blocks of 16 columns; the next product
    reads those and scales its rows: together RMSNorm(x) W2^T, with no norm kernel between. The
    parts are checked one by one, then the whole against the unrounded norm. Widths: no multiple of
    64 (one and four blocks a workgroup both meet an edge), more parts than a thread keeps in
    registers (17024 / 16 > 8 * 32), and the SwiGLU epilogue. Wide second products with K in steps
    of 64 go through the tiled kernel, which finishes the norm in the same way."""
    from herbert_rs_amd.kernels import mfma
    if H in (5120, 5124):        # 320 workgroups of the few-row kernel on 256 CUs: tiles and K slices instead,
        plan = mfma.gemm_plan(M, H, K1, mfma.EPI_ADD, leaves_norm=True)     # and their second kernel leaves the norm
        assert plan > 1000 and plan % 1000 in (112, 124, 184), plan
    a = rand(M, K1, seed=40, dtype=torch.bfloat16)
    w1 = rand(H, K1, seed=41, dtype=torch.bfloat16, scale=0.2)
    x0 = rand(M, H, seed=42, scale=2.0)
    g = 1 + 0.1 * rand(H, seed=43)
    w2 = rand(max(N2, 16), H, seed=44, dtype=torch.bfloat16, scale=0.1)
    eps = 1e-5
    pack = (lambda w: mfma.pack_weight(w)) if packed else (lambda w: w)
    want_x = (x0.double() + a.double() @ w1.double().T).float()
    got_x = x0.clone()
    xg = torch.full((M, H), 7.0, dtype=torch.bfloat16, device=dev())
    blocks = (H + 15) // 16
    MP = mfma.padded_rows(M)
    assert MP >= M and MP < 2 * max(M, 1) and MP & (MP - 1) == 0
    squares = torch.full((blocks, MP), 7.0, device=dev())
    mfma.gemm(a, pack(w1), got_x, accumulate=True, packed=packed, leave=(g, xg, squares, eps))
    assert float((got_x - want_x).abs().max()) <= 2e-6 * K1 ** 0.5 * float(want_x.abs().max()) + 1e-4
    x = got_x                                   # what is left behind is made from the sums as stored
    assert torch.equal(xg, (x * g).to(torch.bfloat16))
    padded = torch.zeros(M, blocks * 16, dtype=torch.float64, device=dev())
    padded[:, :H] = x.double() ** 2
    want_squares = padded.view(M, blocks, 16).sum(-1).T
    assert torch.allclose(squares[:, :M].double(), want_squares, rtol=1e-6, atol=0)
    assert M == MP or float(squares[:, M:].abs().max()) == 0
    if H % 32:
        return          # a width the next product does not take: what was left goes unused

    inv = torch.rsqrt((x.double() ** 2).mean(-1, keepdim=True) + eps)
    want = ((xg.double() @ w2.double().T) * inv).float()
    out = torch.empty(M, N2, device=dev())
    mfma.gemm(xg, pack(w2), out, packed=packed, row_scale=(squares, eps))
    assert float((out - want).abs().max()) <= 1e-5 * float(want.abs().max()) + 1e-5
    exact = ((x.double() * inv * g) @ w2.double().T).float()
    assert float((out - exact).abs().max()) <= 2 ** -7 * float(exact.abs().max())
    if N2 % 32 == 0:
        gate, up = w2[:N2 // 2].contiguous(), w2[N2 // 2:].contiguous()
        wi = mfma.interleave_gate_up(gate, up)
        act = torch.empty(M, N2 // 2, dtype=torch.bfloat16, device=dev())
        mfma.gemm_swiglu(xg, pack(wi), act, packed=packed, row_scale=(squares, eps))
        gg, uu = (xg.double() @ gate.double().T) * inv, (xg.double() @ up.double().T) * inv
        wanted = (gg / (1 + torch.exp(-gg)) * uu).float()
        assert float((act.float() - wanted).abs().max()) <= 2 ** -7 * float(wanted.abs().max()) + 1e-5


@pytest.mark.parametrize("M,H,K,packed", [(17, 64, 512, True), (64, 4096, 4096, True), (40, 1028, 576, False),
                                          (33, 8192, 1024, True), (128, 4096, 4096, True), (300, 2048, 6144, False)])
def test_gemm_mfma_leaves_the_whole_norm_for_more_than_16_rows(M, H, K, packed):
    """K is cut into slices and the kernel that adds them to x norms the rows too: x is the product
    added to what was there, and y the bfloat16 nearest to the norm of that x (or its neighbour).
    Beyond 64 rows this is offered where the product is cut into slices anyway."""
    from herbert_rs_amd.kernels import mfma
    assert mfma.norm_handoff(M, H, K) == "whole"
    a = rand(M, K, seed=45, dtype=torch.bfloat16)
    w = rand(H, K, seed=46, dtype=torch.bfloat16, scale=0.1)
    x0 = rand(M, H, seed=47, scale=2.0)
    g = 1 + 0.1 * rand(H, seed=48)
    eps = 1e-5
    wp = mfma.pack_weight(w) if packed else w
    want_x = (x0.double() + a.double() @ w.double().T).float()
    x = x0.clone()
    y = torch.full((M, H), 7.0, dtype=torch.bfloat16, device=dev())
    mfma.gemm(a, wp, x, accumulate=True, packed=packed, leave=(g, y, None, eps))
    assert float((x - want_x).abs().max()) <= 2e-6 * K ** 0.5 * float(want_x.abs().max()) + 1e-4
    exact = (x.double() * torch.rsqrt((x.double() ** 2).mean(-1, keepdim=True) + eps) * g.double()).float()
    assert float(((y.float() - exact).abs() / exact.abs().clamp_min(1e-3)).max()) <= 2 ** -8 + 1e-4


@pytest.mark.parametrize("tile", [1, 4112, 8112])
def test_gemm_mfma_kernels_by_name_leave_the_same_norm(tile):
    """The few-row kernel (1) and the tiled kernel with K slices, asked for by name, leave the same
    half-done norm behind a product of 8 rows."""
    from herbert_rs_amd.kernels import mfma
    M, H, K = 8, 2048, 2048
    a = rand(M, K, seed=81, dtype=torch.bfloat16)
    w = mfma.pack_weight(rand(H, K, seed=82, dtype=torch.bfloat16, scale=0.1))
    x0 = rand(M, H, seed=83, scale=2.0)
    g = 1 + 0.1 * rand(H, seed=84)
    x = x0.clone()
    xg = torch.empty(M, H, dtype=torch.bfloat16, device=dev())
    squares = torch.empty(H // 16, 8, device=dev())
    mfma.gemm(a, w, x, accumulate=True, packed=True, leave=(g, xg, squares, 1e-6), tile=tile)
    want_x = (x0.double() + a.double() @ rand(H, K, seed=82, dtype=torch.bfloat16, scale=0.1).double().T).float()
    assert float((x - want_x).abs().max()) <= 2e-6 * K ** 0.5 * float(want_x.abs().max()) + 1e-4
    assert torch.equal(xg, (x * g).to(torch.bfloat16))
    want_squares = (x.double() ** 2).view(M, H // 16, 16).sum(-1).T
    assert torch.allclose(squares.double(), want_squares, rtol=1e-6, atol=0)


@pytest.mark.parametrize("M,scaled", [(12, False), (8, True), (16, True), (40, False)])
def test_gemm_mfma_leaves_its_slices_to_the_next_kernel(M, scaled):
    """A plain product whose K is cut leaves the slices' sums in the workspace and says how many
    there are: added up in their order they are the product, bit for bit what the second kernel
    makes of them; a handed-on norm is finished in every slice."""
    from herbert_rs_amd.kernels import mfma
    N, K = 6144, 4096
    a = rand(M, K, seed=90, dtype=torch.bfloat16)
    w = rand(N, K, seed=91, dtype=torch.bfloat16, scale=0.05)
    wp = mfma.pack_weight(w)
    MP = mfma.padded_rows(M)
    squares = (rand(K // 16, MP, seed=92).abs() + 0.5) * 16 if scaled else None
    eps = 1e-6
    row_scale = (squares, eps) if scaled else None
    assert mfma.gemm_plan(M, N, K, finishes_norm=scaled, defer_slices=True) > 1000
    out = torch.full((M, N), 7.0, device=dev())
    n, ptr, stride = mfma.gemm(a, wp, out, packed=True, row_scale=row_scale, defer_slices=True)
    assert n in mfma.DEFERRED_SLICES and stride == M * N and float(out.min()) == 7.0      # out is not written
    parts = torch.empty(n, M, N, device=dev())
    ws = mfma.shared_scratch(dev()).newest_workspace()
    assert ws.data_ptr() == ptr
    parts.copy_(ws[:n * M * N].view(n, M, N))
    whole = torch.empty(M, N, device=dev())
    mfma.gemm(a, wp, whole, packed=True, row_scale=row_scale)
    summed = parts[0].clone()
    for i in range(1, n):
        summed += parts[i]
    want = a.double() @ w.double().T
    if scaled:
        want = want * torch.rsqrt(squares.double().sum(0)[:M, None] / K + eps)
    assert float((summed - want.float()).abs().max()) <= 2e-6 * K ** 0.5 * float(want.abs().max()) + 1e-4
    if mfma.gemm_plan(M, N, K, finishes_norm=scaled) == mfma.gemm_plan(M, N, K, finishes_norm=scaled, defer_slices=True):
        assert torch.equal(summed, whole)


def test_gemm_mfma_refuses_a_handed_norm_it_cannot_do():
    from herbert_rs_amd.errors import BackendError
    from herbert_rs_amd.kernels import mfma
    assert mfma.norm_handoff(16, 64, 32) == "half" and mfma.norm_handoff(17, 64, 32) is None
    assert mfma.norm_handoff(64, 8192, 512) == "whole" and mfma.norm_handoff(2048, 4096, 4096) is None
    assert mfma.norm_handoff(64, 8196, 512) is None and mfma.norm_handoff(20, 64, 448) is None
    M, H = 17, 64
    a = rand(M, 32, seed=1, dtype=torch.bfloat16)
    w = rand(H, 32, seed=2, dtype=torch.bfloat16)
    x = torch.zeros(M, H, device=dev())
    g = torch.ones(H, device=dev())
    xg = torch.empty(M, H, dtype=torch.bfloat16, device=dev())
    squares = torch.empty(4, 4, device=dev())
    eps = 1e-6
    with pytest.raises(BackendError):
        mfma.gemm(a, w, x, accumulate=True, leave=(g, xg, squares, eps))            # more than 16 rows
    with pytest.raises(BackendError):
        mfma.gemm(a, w, x, accumulate=True, leave=(g, xg, None, eps))               # K too short to cut
    with pytest.raises(BackendError):
        mfma.gemm(a[:4], w, x[:4], accumulate=False, leave=(g, xg[:4], squares, eps))    # nothing is added
    with pytest.raises(BackendError):
        mfma.gemm(xg[:4], rand(32, H, seed=3, dtype=torch.bfloat16), torch.zeros(4, 32, device=dev()),
                  accumulate=True, row_scale=(squares, 1e-6))


# every tile with every size it takes (K in steps of 32 goes to the host's own choice and to tile 123 only)
TILE_CASES = [(tile, M, N, K, packed)
              for tile in (0, 188, 142, 186, 122, 123, 112, 124, 184)
              for M, N, K, packed in [(65, 128, 64, True), (200, 336, 192, True), (300, 530, 96, False),
                                      (513, 1040, 256, True), (2300, 528, 128, True), (17, 272, 64, True),
                                      (40, 530, 320, False), (64, 1040, 128, True)]
              if K % 64 == 0 or tile in (0, 123)]


@pytest.mark.parametrize("tile,M,N,K,packed", TILE_CASES)
def test_gemm_mfma_tile_variants(tile, M, N, K, packed):
    from herbert_rs_amd.kernels import mfma
    a = rand(M, K, seed=7, dtype=torch.bfloat16)
    w = rand(N, K, seed=8, dtype=torch.bfloat16)
    want = (a.double() @ w.double().T).float()
    wp = mfma.pack_weight(w) if packed else w
    c = torch.full((M, N), 7.0, device=dev())
    mfma.gemm(a, wp, c, packed=packed, tile=tile)
    tol = 2e-6 * K ** 0.5 * float(want.abs().max()) + 1e-4
    assert float((c - want).abs().max()) <= tol
    base = rand(M, N, seed=9)
    c2 = base.clone()
    mfma.gemm(a, wp, c2, accumulate=True, packed=packed, tile=tile)
    assert float((c2 - (base + want)).abs().max()) <= tol
    if N % 32 == 0:
        gate, up = w[:N // 2].contiguous(), w[N // 2:].contiguous()
        wi = mfma.interleave_gate_up(gate, up)
        out = torch.empty(M, N // 2, dtype=torch.bfloat16, device=dev())
        mfma.gemm_swiglu(a, mfma.pack_weight(wi) if packed else wi, out, packed=packed, tile=tile)
        g, u = a.double() @ gate.double().T, a.double() @ up.double().T
        wanted = (g / (1 + torch.exp(-g)) * u).float()
        assert float((out.float() - wanted).abs().max()) <= 2 ** -7 * float(wanted.abs().max()) + 1e-4


def _slices_fit(tile, K):
    """A tile number's slices (its thousands) are no more than the workspace is sized for and leave no slice empty."""
    slices, steps = tile // 1000, K // 64
    return slices <= 1 or (slices <= min(16, K // 256) and -(-steps // slices) * (slices - 1) < steps)


SLICE_CASES = [(tile, M, N, K, packed)
               for tile in (0, 2122, 4188, 3142, 2186, 8122, 4112, 16124, 2184)
               for M, N, K, packed in [(200, 336, 512, True), (513, 1040, 768, True), (128, 1024, 4096, True),
                                       (300, 530, 1024, False), (24, 1056, 2112, True), (64, 8192, 1024, True),
                                       (33, 336, 4096, False)]
               if _slices_fit(tile, K)]


@pytest.mark.parametrize("tile,M,N,K,packed", SLICE_CASES)
def test_gemm_mfma_tiled_with_k_slices(tile, M, N, K, packed):
    """Few tiles: K is cut into slices over workgroups (thousands of the tile number = slices), the
    sums added in order by a second kernel, also under the SwiGLU epilogue; tile 0 chooses by
    itself (K = 2112 = 33 steps: eight slices of five steps would leave the last one empty)."""
    from herbert_rs_amd.kernels import mfma
    a = rand(M, K, seed=60, dtype=torch.bfloat16)
    w = rand(N, K, seed=61, dtype=torch.bfloat16, scale=0.05)
    want = (a.double() @ w.double().T).float()
    wp = mfma.pack_weight(w) if packed else w
    tol = 2e-6 * K ** 0.5 * float(want.abs().max()) + 1e-4
    c = torch.full((M, N), 7.0, device=dev())
    mfma.gemm(a, wp, c, packed=packed, tile=tile)
    assert float((c - want).abs().max()) <= tol
    base = rand(M, N, seed=62)
    c2 = base.clone()
    mfma.gemm(a, wp, c2, accumulate=True, packed=packed, tile=tile)
    assert float((c2 - (base + want)).abs().max()) <= tol
    c3 = base.clone()
    mfma.gemm(a, wp, c3, accumulate=True, packed=packed, tile=tile)
    assert torch.equal(c2, c3)          # the slices are added in a fixed order
    if N % 32 == 0:
        gate, up = w[:N // 2].contiguous(), w[N // 2:].contiguous()
        wi = mfma.interleave_gate_up(gate, up)
        out = torch.full((M, N // 2), 7.0, dtype=torch.bfloat16, device=dev())
        mfma.gemm_swiglu(a, mfma.pack_weight(wi) if packed else wi, out, packed=packed, tile=tile)
        g, u = a.double() @ gate.double().T, a.double() @ up.double().T
        wanted = (g / (1 + torch.exp(-g)) * u).float()
        assert float((out.float() - wanted).abs().max()) <= 2 ** -7 * float(wanted.abs().max()) + 1e-4


@pytest.mark.parametrize("M,N,K", [(17, 4096, 4096), (40, 1024, 512), (64, 4096, 12288), (64, 6144, 4096),
                                   (33, 272, 96)])
def test_gemm_mfma_with_k_slices(M, N, K):
    """17 to 64 rows: K is cut into slices over several workgroups whose sums a second kernel adds."""
    from herbert_rs_amd.kernels import mfma
    a = rand(M, K, seed=40, dtype=torch.bfloat16)
    w = rand(N, K, seed=41, dtype=torch.bfloat16, scale=0.05)
    want = (a.double() @ w.double().T).float()
    tol = 2e-6 * K ** 0.5 * float(want.abs().max()) + 1e-4
    for packed in (False, True):
        wp = mfma.pack_weight(w) if packed else w
        c = torch.full((M, N), 3.0, device=dev())
        mfma.gemm(a, wp, c, packed=packed)
        assert float((c - want).abs().max()) <= tol
        base = rand(M, N, seed=42)
        c2 = base.clone()
        mfma.gemm(a, wp, c2, accumulate=True, packed=packed)
        assert float((c2 - (base + want)).abs().max()) <= tol
        c3 = base.clone()
        mfma.gemm(a, wp, c3, accumulate=True, packed=packed)
        assert torch.equal(c2, c3)                      # the same bits on every run


# ---------------------------------------------------------------- random weights
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n,first", [(1, 0), (255, 7), (256, 0), (100003, 12345), (1 << 20, (1 << 33) + 5)])
def test_random_fill_on_the_gpu_is_the_hosts(dtype, n, first):
    """The kernel that draws weights on the GPU and the host's threads compute one function: the same
    bits for any count, any first index (also beyond 2^32), as float32 and as bfloat16, with and without
    an offset; and against the formula itself for the first values."""
    from herbert_rs_amd.weights import random_init as ri
    from .test_config_weights import counter_values
    key = 0x0123456789ABCDEF ^ n
    for scale, offset in ((0.02 / ri.BYTE_SUM_SIGMA, 0.0), (0.1 / ri.BYTE_SUM_SIGMA, 1.0)):
        on_gpu = ri.counter_fill(torch.empty(n, dtype=dtype, device=dev()), key, scale, offset, first=first)
        on_host = ri.counter_fill(torch.empty(n, dtype=dtype), key, scale, offset, first=first)
        assert torch.equal(on_gpu.cpu(), on_host)
        want = counter_values(key, first, min(n, 50), scale, offset)
        assert np.array_equal(on_host[:50].float().numpy(), torch.tensor(want).to(dtype).float().numpy())
