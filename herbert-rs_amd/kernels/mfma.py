"""Host side of the bfloat16 MFMA kernels (matrix products and attention): which shapes they
take, operand checks, launches. What they refuse goes to the plain kernels.

The reference rounds the inputs of its bfloat16 product to bfloat16 and sums in float32 as well
(crates/backends/backend_bf16_avx512/src/avx512_bf16_matvec.S:1-12); its GPU backend chooses between a
single-pass and a split decode attention by the context's length
(crates/backends/backend_metal/src/kernels/attention.rs:73-91), as _decode_split does here."""
import ctypes

import torch

from ..errors import BackendError
from . import lib
from .ops import _check, _stream

_P = ctypes.c_void_p
_I = ctypes.c_int
_F = ctypes.c_float
lib.register_signatures("gemm_mfma", {
    "hb_gemm_mfma": [_P, _P, _P, _I, _I, _I, _I, _I, _I, _P, _F, _I, _P, ctypes.c_size_t, _P, _P, _P, _P, _I, _F,
                     _F, _P, _P],
    "hb_gemm_mfma_plan": [_I, _I, _I, _I, _I, _I, _I, ctypes.c_size_t, _I],
    "hb_gemm_mfma_plan_cost": [_I, _I, _I, _I, _I, _I, _I, ctypes.c_size_t, _I],
    "hb_gemm_mfma_split": [_I, _I, _I, _I, ctypes.c_size_t],
    "hb_gemm_qkv_mfma": [_P, _P, _I, _I, _I, _P, _P, _P, _P, _P, _P, _P, _I, _I, _P, _P, _P, _P, _F, _I, _I, _I, _I, _P],
})

EPI_STORE, EPI_ADD, EPI_SWIGLU = 0, 1, 2
SLICE_WORKSPACE_FLOATS = 16 << 20     # most that the tiled product may use for its K slices (64 MB)


class Scratch:
    """The device memory that these kernels use beyond their operands, for one owner: the workspace
    of products whose K is cut into slices, and the partial results of the decode attention's
    ranges. An engine's Runtime owns one, so that two engines of a process (each on a stream of its
    own) never write the same scratch; callers without an owner (tests, measurements) share one a
    device. A buffer that was handed out is kept for good, also when a larger one replaces it: a
    captured graph may hold its address."""

    def __init__(self):
        self.workspaces = []         # float32 buffers, the newest and largest last
        self.workspace_of = {}       # (device, M, N, K, tile) -> (pointer, floats)
        self.partials = []           # (outputs, maxima and sums) of the decode attention's ranges

    def newest_workspace(self):
        return self.workspaces[-1] if self.workspaces else None


def _not_while_recording(what):
    """Nothing is allocated while a step is recorded into a graph: the step runs outside one first."""
    if torch.cuda.is_current_stream_capturing():
        from ..errors import NeedsEagerStep
        raise NeedsEagerStep(f"{what} would have to be allocated while a graph is recorded")


_shared_scratch = {}


def _scratch_of(scratch, device):
    if scratch is not None:
        return scratch
    device = torch.device(device)
    if device.index is None:
        device = torch.device(device.type, torch.cuda.current_device())
    found = _shared_scratch.get(device)
    if found is None:
        found = _shared_scratch[device] = Scratch()
    return found


def shared_scratch(device):
    """The Scratch of callers that bring none, for `device`."""
    return _scratch_of(None, device)


def _slice_workspace_floats(M, N, K, tile=0):
    """The floats of scratch that a product of these sizes is given for its K slices (0: it is never
    cut): room for as many slices as the kernel's estimate may choose, up to SLICE_WORKSPACE_FLOATS.
    Only products with few tiles are cut (whether, and how, is the kernel's estimate)."""
    tiles = ((M + 255) // 256) * ((N + 255) // 256)       # of the largest kind: under two rounds of them on 256 CUs
    slices = min(16, K // 256) if tiles < 512 or tile else 1
    # (a product too large to be cut even in two still gets the room: where its rows are cut into
    # whole tiles and a rest, the rest's few rows are cut along K)
    return min(slices * M * N, SLICE_WORKSPACE_FLOATS) if slices >= 2 else 0


def _slice_workspace(scratch, device, M, N, K, tile=0):
    """(pointer, floats) of the scratch for a product whose K may be cut into slices."""
    scratch = _scratch_of(scratch, device)
    key = (device, M, N, K, tile)
    found = scratch.workspace_of.get(key)           # (a buffer that was handed out stays valid)
    if found is not None:
        return found
    need = _slice_workspace_floats(M, N, K, tile)
    if need == 0:
        found = (None, 0)
    else:
        kept = scratch.workspaces
        if not kept or kept[-1].numel() < need:
            _not_while_recording("the workspace of a product's K slices")
            kept.append(torch.empty(need, dtype=torch.float32, device=device))
        found = (kept[-1].data_ptr(), kept[-1].numel())
    if len(scratch.workspace_of) > 4096:
        scratch.workspace_of.clear()
    scratch.workspace_of[key] = found
    return found


def gemm_supported(a, w, out=None, swiglu=False):
    """True if hb_gemm_mfma takes this product (bfloat16 operands, K in steps of 32; the SwiGLU
    epilogue pairs blocks of 16 rows)."""
    if a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        return False
    M, K = a.shape
    N = w.shape[0]
    if K % 32:
        return False
    if swiglu:
        return N % 32 == 0
    return out is None or out.dtype == torch.float32


def pack_weight(w):
    """[N, K] -> the same values as [K / 32, N / 16, 64, 8]: the 1 KB MFMA operand of 16 rows and
    32 k is contiguous, lane-major (lane = 16 * (k / 8 % 4) + n % 16), and the operands of one
    k-step lie together, so that workgroups advancing through K side by side read memory as a
    streaming copy does."""
    N, K = w.shape
    if N % 16 or K % 32:
        raise BackendError("packed weights need N in steps of 16 and K in steps of 32")
    return w.view(N // 16, 16, K // 32, 4, 8).permute(2, 0, 3, 1, 4).contiguous().view(N, K)


def _norm_args(a, norm, K):
    """(pointer, eps) of a fused RMSNorm, after checks; (None, 0) without one."""
    if norm is None:
        _check(a, "a", torch.bfloat16, (None, None))
        return None, 0.0
    weight, eps = norm
    _check(a, "a", torch.float32, (None, None))
    _check(weight, "norm weight", torch.float32, (K,))
    if a.shape[0] > NORM_FUSE_MAX_M:
        raise BackendError(f"the fused norm takes at most {NORM_FUSE_MAX_M} rows")
    return weight.data_ptr(), float(eps)


NORM_FUSE_MAX_M = 16
NORM_FUSE_MIN_N = 16384     # measured: for narrower products a norm kernel of its own is as fast or faster


def norm_fusable(a, w):
    """True if RMSNorm(a) @ w^T should run as one kernel: at most 16 rows of the float32 residual
    stream (every workgroup reads all of them; with more rows that costs more than a norm kernel)
    and many weight rows (each workgroup then has enough of them to pay for reading the rows)."""
    return (a.dtype == torch.float32 and w.dtype == torch.bfloat16 and a.shape[0] <= NORM_FUSE_MAX_M
            and a.shape[1] % 32 == 0 and w.shape[0] >= NORM_FUSE_MIN_N)


NORM_HANDOFF_MAX_M = 16


def padded_rows(M):
    """The rows of a handed-on norm's sums of squares: M rounded up to a power of two."""
    return 1 << max(0, int(M) - 1).bit_length()


NORM_WHOLE_MAX_M = 64         # up to here a product that leaves a norm behind is cut into K slices for it
NORM_WHOLE_MAX_N = 8192


_handoffs = {}


def norm_handoff(M, N, K):
    """See _norm_handoff; the answer for a size is worked out once."""
    key = (M, N, K)
    how = _handoffs.get(key, 0)
    if how == 0:
        how = _handoffs[key] = _norm_handoff(M, N, K)
    return how


def _norm_handoff(M, N, K):
    """How a product of these sizes that adds to the residual stream can prepare the RMSNorm that
    follows: "half" (at most 16 rows: bf16(x * g) and sums of squares, finished by the next product),
    "whole" (more rows: the kernel that adds up the K slices norms the rows too; beyond 64 rows only
    if the product is cut into slices anyway) or None."""
    if K % 32:
        return None
    if M <= NORM_HANDOFF_MAX_M:
        return "half"
    if K % 64 == 0 and K >= 512 and N % 4 == 0 and N <= NORM_WHOLE_MAX_N:
        if M <= NORM_WHOLE_MAX_M or gemm_plan(M, N, K, EPI_ADD) >= 2000:
            return "whole"
        # Not cut by itself: cut it for the norm's sake if that is estimated to take less time than the
        # uncut product and a norm kernel (one read of the float32 rows, one write of bfloat16 ones).
        alone, cut = gemm_plan_cost(M, N, K, EPI_ADD), gemm_plan_cost(M, N, K, EPI_ADD, leaves_norm=True)
        if alone > 0 and cut > 0 and cut < alone + 2.3 + M * N * 6 / 5.0e6:
            return "whole"
    return None


def _handoff_args(M, N, K, leave, row_scale, accumulate, norm):
    """The seven arguments of a norm that is handed from one product to the next, after checks.
    leave = (norm weight f32 [N], xg bf16 [M, N], squares f32 [ceil(N / 16), padded_rows(M)], eps): the
    product adds to the residual stream and leaves bf16(x * weight) and the sums of x^2 over blocks
    of 16 columns; with squares = None (17 to 64 rows) it leaves the whole norm in xg.
    row_scale = (squares f32 [ceil(K / 16), padded_rows(M)], eps): the input is such an xg, and every
    row of the product is scaled by 1 / sqrt(sum of its squares / K + eps)."""
    args = [None, None, None, None, 0, 0.0, 0.0]
    if leave is None and row_scale is None:
        return args
    if norm is not None:
        raise BackendError("a norm is never handed on beside a fused one")
    if leave is not None:
        weight, xg, squares, eps = leave
        how = norm_handoff(M, N, K)
        if not accumulate or how != ("half" if squares is not None else "whole"):
            raise BackendError(f"a product of M={M}, N={N}, K={K} cannot leave this norm behind")
        _check(weight, "norm weight", torch.float32, (N,))
        _check(xg, "xg", torch.bfloat16, (M, N))
        args[:2] = [weight.data_ptr(), xg.data_ptr()]
        args[6] = float(eps)
        if squares is not None:
            _check(squares, "squares", torch.float32, ((N + 15) // 16, padded_rows(M)))
            args[2] = squares.data_ptr()
    if row_scale is not None:
        squares, eps = row_scale
        if accumulate or M > NORM_HANDOFF_MAX_M:
            raise BackendError("a handed-on norm is finished by a product of at most 16 rows that does not add")
        _check(squares, "squares", torch.float32, ((K + 15) // 16, padded_rows(M)))
        args[3:6] = [squares.data_ptr(), squares.shape[0], float(eps)]
    return args


def gemm_plan(M, N, K, epi=EPI_STORE, normed_input=False, leaves_norm=False, finishes_norm=False, device=None,
              defer_slices=False):
    """Which kernel hb_gemm_mfma picks for a product, for tests and measurements: 0 = the few-row
    kernel, otherwise the tile variant + 1000 x the K slices (if more than one), -1 = refused. The
    choice is the host's and needs no GPU (`device` is not used): more scratch than a product is
    given by _slice_workspace_floats never changes it, since that is room for every number of
    slices the estimate considers."""
    ws_floats = _slice_workspace_floats(M, N, K)
    return lib.load("gemm_mfma").hb_gemm_mfma_plan(M, N, K, epi, int(normed_input), int(leaves_norm),
                                                   int(finishes_norm), ws_floats, int(defer_slices))


def gemm_split(M, N, K, epi=EPI_STORE, device=None):
    """The rows that hb_gemm_mfma cuts off as a first product of their own (whole tiles; the rest
    follows as a second product), or 0 where it runs the product whole."""
    ws_floats = _slice_workspace_floats(M, N, K)
    return lib.load("gemm_mfma").hb_gemm_mfma_split(M, N, K, epi, ws_floats)


def gemm_plan_cost(M, N, K, epi=EPI_STORE, normed_input=False, leaves_norm=False, finishes_norm=False, device=None,
                   defer_slices=False):
    """The estimated time in us of the plan gemm_plan gives; negative where no estimate chose it."""
    ws_floats = _slice_workspace_floats(M, N, K)
    fn = lib.load("gemm_mfma").hb_gemm_mfma_plan_cost
    fn.restype = ctypes.c_double
    return fn(M, N, K, epi, int(normed_input), int(leaves_norm), int(finishes_norm), ws_floats, int(defer_slices))


def gemm(a, w, out, accumulate=False, packed=False, norm=None, tile=0, leave=None, row_scale=None,
         defer_slices=False, scratch=None):
    """out f32 [M, N] (+)= a bf16 [M, K] @ w bf16 [N, K]^T (w as stored, or as pack_weight gives it).
    norm = (weight f32 [K], eps): a is the float32 residual stream and is RMS-normed on the way.
    leave, row_scale: see _handoff_args.
    defer_slices: if the kernel cuts K into slices it leaves their sums for the caller's next kernel
    to add up; returns (slices, pointer to the first, floats between two): with slices == 1 `out`
    holds the product as usual, otherwise `out` is not written.
    scratch: the caller's Scratch (the K slices' workspace comes from it); None: the device's shared one."""
    M, K = a.shape
    norm_ptr, eps = _norm_args(a, norm, K)
    _check(w, "w", torch.bfloat16, (None, K))
    N = w.shape[0]
    _check(out, "out", torch.float32, (M, N))
    if K % 32 or (norm is not None and accumulate):
        raise BackendError(f"gemm_mfma refuses M={M}, N={N}, K={K}")
    hand = _handoff_args(M, N, K, leave, row_scale, accumulate, norm)
    ws_ptr, ws_floats = _slice_workspace(scratch, a.device, M, N, K, tile)
    if defer_slices and (accumulate or leave is not None):
        raise BackendError("only a plain product leaves its slices to the next kernel")
    deferred = ctypes.c_int(1) if defer_slices else None
    lib.call("gemm_mfma", "hb_gemm_mfma", a.data_ptr(), w.data_ptr(), out.data_ptr(), M, N, K, N,
             EPI_ADD if accumulate else EPI_STORE, 1 if packed else 0, norm_ptr, eps, int(tile), ws_ptr,
             ws_floats, *hand, ctypes.byref(deferred) if defer_slices else None, _stream())
    if defer_slices:
        return (deferred.value, ws_ptr, M * N) if deferred.value > 1 else (1, out.data_ptr(), 0)
    return None


QKV_FUSE_MIN_TILES = 136   # of 256 x 256; with fewer (measured: 120 lose, 144 win) the plain product's smaller tiles or K slices fill the CUs better


def qkv_tile_shape(M, N):
    """The tiles on which a q/k/v projection of M rows and N = heads x 128 columns norms, rotates and
    writes the cache itself, or None where it should not (too few tiles to fill the CUs: the plain
    product's smaller tiles and K slices then do better, and a kernel of its own does the rest).
    0: 256 x 256; 1: a head wide, 256 rows high; 2: a head wide, 128 rows high."""
    tiles = -(-M // 256) * -(-N // 256)
    if tiles >= QKV_FUSE_MIN_TILES:
        # (rows that end a little past whole tiles, with a last round of tiles that is nearly empty:
        # the plain product cuts such rows off as a product of their own and is then ahead, 3 % of a
        # prompt of 2,600 tokens)
        if tiles > 256 and tiles % 256 < 64 and 0 < M % 256 <= 64:
            return None
        return 0
    heads = N // 128
    for shape, rows in ((1, 256), (2, 128)):
        if QKV_FUSE_MIN_TILES <= -(-M // rows) * heads <= 256:
            return shape
    return None


def gemm_qkv_fusable(a, w, meta, kv, nq, nkv, hd, rot_dims):
    """True if the q/k/v projection of this step should norm, rotate and write the cache itself:
    a long enough bfloat16 prompt step, heads of 128 rotated whole or not at all, pages of 64 tokens."""
    return (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and kv.k.dtype == torch.bfloat16
            and a.shape[1] % 64 == 0 and hd == 128 and kv.page_size == 64
            and rot_dims in (0, hd) and w.shape[0] == (nq + 2 * nkv) * hd and meta.num_tokens == a.shape[0]
            and qkv_tile_shape(a.shape[0], w.shape[0]) is not None)


def gemm_qkv(a, w, packed, q_norm_w, k_norm_w, cos, sin, meta, kv, q_out, nq, nkv, hd, eps, shape=None):
    """q_out bf16 [M, nq hd] and the pages of kv from a bf16 [M, K] @ w[(nq + 2 nkv) hd, K]^T: the
    product, the per-head norm (if weights are given), the rotation (if tables are given) and the
    cache write in one kernel. `shape`: the tiles (see qkv_tile_shape), by default what that picks
    or, where it picks none, the large ones."""
    M, K = a.shape
    if shape is None:
        shape = qkv_tile_shape(M, (nq + 2 * nkv) * hd) or 0
    _check(a, "a", torch.bfloat16, (M, K))
    _check(w, "w", torch.bfloat16, ((nq + 2 * nkv) * hd, K))
    _check(q_out, "q_out", torch.bfloat16, (M, nq * hd))
    pages = kv.k.shape[0]
    _check(kv.k, "key pages", torch.bfloat16, (pages, nkv, 64, hd))
    _check(kv.v, "value pages", torch.bfloat16, (pages, nkv, hd, 64))
    _check(kv.page_table, "page_table", torch.int32, (None, None))
    _check(meta.positions, "positions", torch.int32, (M,))
    _check(meta.seq_of, "seq_of", torch.int32, (M,))
    _check(meta.slots, "slots", torch.int32, (meta.num_seqs,))
    if hd != 128 or K % 64:
        raise BackendError(f"the fused q/k/v product refuses head_dim {hd}, K={K}")
    for t, name in ((q_norm_w, "q_norm"), (k_norm_w, "k_norm")):
        if t is not None:
            _check(t, name, torch.float32, (hd,))
    if (cos is None) != (sin is None):
        raise BackendError("cos and sin tables come together")
    if cos is not None:
        _check(cos, "cos", torch.float32, (None, hd // 2))
        _check(sin, "sin", torch.float32, tuple(cos.shape))
        if meta.max_position >= cos.shape[0]:
            raise BackendError(f"position {meta.max_position} beyond the rotation table ({cos.shape[0]} rows)")
    ptr = lambda t: None if t is None else t.data_ptr()
    lib.call("gemm_mfma", "hb_gemm_qkv_mfma", a.data_ptr(), w.data_ptr(), M, K, 1 if packed else 0, q_out.data_ptr(),
             kv.k.data_ptr(), kv.v.data_ptr(), meta.positions.data_ptr(), meta.seq_of.data_ptr(),
             meta.slots.data_ptr(), kv.page_table.data_ptr(), kv.page_table.shape[1], kv.page_size, ptr(q_norm_w),
             ptr(k_norm_w), ptr(cos), ptr(sin), float(eps), nq, nkv, hd, int(shape), _stream())


def interleave_gate_up(gate, up):
    """[2I, K] with blocks of 16 gate rows followed by the 16 up rows of the same outputs:
    the row order the SwiGLU epilogue expects."""
    I, K = gate.shape
    if I % 16 or up.shape != gate.shape:
        raise BackendError("gate and up must have the same shape with rows in steps of 16")
    return torch.stack([gate.view(I // 16, 16, K), up.view(I // 16, 16, K)], 1).reshape(2 * I, K).contiguous()


def gemm_swiglu(a, w_interleaved, out, packed=False, norm=None, tile=0, row_scale=None, scratch=None):
    """out bf16 [M, I] = silu(a @ gate^T) * (a @ up^T), the weights interleaved as above.
    row_scale: see _handoff_args (gate and up are scaled before the activation)."""
    M, K = a.shape
    norm_ptr, eps = _norm_args(a, norm, K)
    _check(w_interleaved, "w", torch.bfloat16, (None, K))
    N = w_interleaved.shape[0]
    _check(out, "out", torch.bfloat16, (M, N // 2))
    if K % 32 or N % 32:
        raise BackendError(f"gemm_mfma (SwiGLU) refuses M={M}, N={N}, K={K}")
    hand = _handoff_args(M, N, K, None, row_scale, False, norm)
    ws_ptr, ws_floats = _slice_workspace(scratch, a.device, M, N, K, tile)
    lib.call("gemm_mfma", "hb_gemm_mfma", a.data_ptr(), w_interleaved.data_ptr(), out.data_ptr(), M, N, K,
             N // 2, EPI_SWIGLU, 1 if packed else 0, norm_ptr, eps, int(tile), ws_ptr, ws_floats, *hand, None,
             _stream())


lib.register_signatures("attention_mfma", {
    "hb_attn_prefill_mfma": [_P, _P, _P, _P, _P, _P, _P, _I, _P, _P, _P, _I, _I, _I, _I, _I, _F, _I, _I, _P],
    "hb_attn_decode_mfma": [_P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _F, _I, _I, _I,
                            _P, _P, _P, _P, _P, _F, _I, _I, ctypes.c_size_t, _P, _P],
})

ATTENTION_HEAD_DIMS = (32, 64, 128)
QUERY_TILE = 32


def attention_supported(q, kv, nq, nkv, hd):
    """bfloat16, pages of 64 tokens, a head size the kernels are built for, at most 32 query heads
    to a kv head."""
    return (q.dtype == torch.bfloat16 and kv.k.dtype == torch.bfloat16 and kv.page_size == 64
            and hd in ATTENTION_HEAD_DIMS and nq % nkv == 0 and nq // nkv <= 32)


PREFILL_LONG_MIN_WORKGROUPS = 512      # from so many workgroups of 64-token tiles on (measured: 4 K tokens of 8 kv heads 200 -> 176 us, 2 K 57 -> 70): the kernel for long prompts


def _prefill_tile_height(meta, nkv, group):
    """32, or 64 where the step has so many tokens that tiles of 64 still make several rounds of
    workgroups: the kernel for those loads every page once for 64 tokens and has its loads two
    steps ahead; with fewer, tiles of 32 whose pages two groups of waves take in turn end sooner.
    Tiles of 64 must be worth their eight waves: those of at most 32 tokens (single tokens of
    running sequences beside a prompt, a prompt's short end) leave one half idle and walk their
    pages alone, so a step made mostly of them keeps tiles of 32."""
    key = ("prefill_tile_height", nkv, group)
    height = meta.derived.get(key)          # every layer's attention asks: worked out once a step
    if height is None:
        height = meta.derived[key] = _prefill_tile_height_of(meta, nkv, group)
    return height


def _prefill_tile_height_of(meta, nkv, group):
    tiles = full = 0
    for i in range(meta.num_seqs):
        n = int(meta.host_starts[i + 1]) - int(meta.host_starts[i])
        tiles += -(-n // 64)
        full += n // 64 + (1 if n % 64 > 32 else 0)
    per_tile = nkv * -(-group // 4)
    return 64 if full * per_tile >= PREFILL_LONG_MIN_WORKGROUPS and 4 * full >= 3 * tiles else 32


def _prefill_tiles(meta, height=QUERY_TILE):
    """Device arrays (sequence, first packed row, rows) of the query tiles of a step (`height` tokens
    each), those that see the most keys first: the kernel deals them out heaviest first."""
    tiles = meta.derived.get(("prefill_tiles", height))
    if tiles is None:
        items = []
        starts, context = meta.host_starts, meta.host_context
        for i in range(meta.num_seqs):
            a, b = int(starts[i]), int(starts[i + 1])
            for r in range(a, b, height):
                n = min(height, b - r)
                last_position = int(context[i]) - (b - (r + n)) - 1
                items.append((-last_position, i, r, n))
        items.sort()
        seq, row0, rows = [it[1] for it in items], [it[2] for it in items], [it[3] for it in items]
        packed = torch.tensor([seq, row0, rows], dtype=torch.int32).to(meta.positions.device)
        tiles = (packed[0], packed[1], packed[2], len(seq))
        meta.derived[("prefill_tiles", height)] = tiles
    return tiles


DECODE_WAVES = 1024       # waves of the decode kernel that the 256 CUs hold at a time


def _decode_split(meta, nkv, window):
    """(ranges, pages per range): as many ranges as still give no more waves than the GPU holds at
    a time, every range at least one page. With one range the kernel writes the output itself and
    no merge runs. (Measured at 4 K tokens a sequence: what costs is a second, partly filled round
    of waves. 48 sequences x 8 kv heads: 2 ranges, 768 waves, 9.8 ms a step; 3 ranges, 1152 waves,
    10.6 ms. 40 sequences: 3 ranges, 960 waves, 8.9 ms; 4 ranges, 1280 waves, 10.0 ms.)"""
    span = (meta.context_bucket + 63) // 64     # by bucket, so that a captured graph's grid stays right
    if window:
        span = min(span, (window + 63) // 64 + 1)
    pairs = meta.num_seqs * nkv
    if 2 * pairs >= DECODE_WAVES:
        # (how evenly the waves sit is a matter of the sequences themselves: padding rows' waves end at once)
        pairs = (getattr(meta, "num_real", 0) or meta.num_seqs) * nkv
        # Two waves a CU already: a merge costs more than it gains (5 to 8 % of a step), as long as
        # the waves sit evenly. A wave that reads a whole context is a long job, and the time goes
        # with the CU that has the most of them (three where most have two: 65 sequences took a
        # quarter longer than 64) or, beyond what the GPU holds at a time, with the last round
        # (160 sequences: two rounds for one and a quarter). Where the most is 1.3 times the mean
        # or more, eight ranges (four for contexts under 2 K tokens, none under 1 K) even that out:
        # 7 % off at 65 sequences, 10 to 12 % at 136 to 160.
        unit = max(1, DECODE_WAVES // 4) if pairs <= DECODE_WAVES else DECODE_WAVES     # what fills evenly
        fine = min(8, span // 4)
        if -(-pairs // unit) >= 1.3 * pairs / unit and fine >= 4:
            per = -(-span // fine)
            return -(-span // per), per
        return 1, span
    # the merge's cost grows with the ranges: more than 32 only where each still has four pages
    most = max(1, min(span, max(32, min(128, span // 4))))
    best = (1, span)
    for cand in range(2, most + 1):
        per = -(-span // cand)
        ranges = -(-span // per)
        if pairs * ranges <= DECODE_WAVES and ranges > best[0]:
            best = (ranges, per)
    return best


def _decode_ranges(meta, nkv, window):
    """(items of the grid, list of ranges on the GPU) for a step whose contexts are of very unequal
    lengths, else None. Equal shares would leave the waves of the short sequences with nothing and
    those of the long ones with all the work (one sequence of 32 K tokens beside seven of 1 K: 128 of
    1,024 waves read 2 K tokens each); with the list every wave has a range of the same length of
    whichever sequence, as many ranges as the GPU holds waves at a time (more where that would be
    fewer than two a sequence, and the lengths are unequal enough for more than one round of waves
    to pay). The list changes with every step and is read by the kernel; the grid does not change."""
    B = meta.num_seqs
    if not meta.unequal or window or B < 2 or meta.max_new != 1:
        return None
    # at least two items a sequence, so that a range is no longer than the mean sequence: beyond
    # half a round of sequences the grid is more than one round of waves (the kernel's limit: 1,024 items)
    items = max(DECODE_WAVES // nkv, 2 * B)
    if items > 1024 or items < 4 or (items * nkv > DECODE_WAVES and meta.unequal < 2):
        return None
    listed = meta.ranges_for(items, 64)
    return None if listed is None else (items, listed)


def _partial_buffers(scratch, device, n_rows, splits, hd):
    """(partial outputs, partial max / sum) of the decode kernel's ranges, from the caller's Scratch.
    Buffers that were handed out are kept for good, also when larger ones replace them: a captured
    graph may hold their addresses."""
    kept = _scratch_of(scratch, device).partials
    need_o, need_ml = n_rows * splits * hd, n_rows * splits * 2
    if not kept or kept[-1][0].numel() < need_o or kept[-1][1].numel() < need_ml:
        _not_while_recording("the decode attention's partial results")
        grow = 2 if kept else 1
        kept.append((torch.empty(max(need_o, grow * (kept[-1][0].numel() if kept else 0)), dtype=torch.float32,
                                 device=device),
                     torch.empty(max(need_ml, grow * (kept[-1][1].numel() if kept else 0)), dtype=torch.float32,
                                 device=device)))
    return kept[-1]


def decode_fusable(meta, kv, nq, nkv, hd, rot_dims, dtype):
    """True if the decode kernel can do the per-head norm, the rotation and the cache write itself:
    one token a sequence, bfloat16, a head size it is built for, rotation over the whole head or none."""
    return (meta.max_new == 1 and meta.num_tokens == meta.num_seqs and dtype == torch.bfloat16
            and kv.k.dtype == torch.bfloat16 and kv.page_size == 64 and hd in ATTENTION_HEAD_DIMS
            and nq % nkv == 0 and nq // nkv <= 32 and rot_dims in (0, hd))


def attention_decode_fused(qkv, q_norm_w, k_norm_w, cos, sin, meta, kv, out, nq, nkv, hd, eps, scale, window,
                           qkv_slices=None, scratch=None):
    """One token a sequence: per-head norm (if weights are given), rotation (if tables are given),
    the new key and value written to the pages, and attention over them, in one kernel (+ merge).
    qkv f32 [B, (nq + 2 nkv) hd]; cos / sin f32 [max_pos, hd / 2]; out bf16 [B, nq hd].
    qkv_slices = (slices, pointer, floats between two), as gemm(..., defer_slices=True) returns it:
    the projection's sums are still in that many slices, which the kernel adds up as it loads them
    (qkv itself is then not read)."""
    B = meta.num_seqs
    _check(qkv, "qkv", torch.float32, (B, (nq + 2 * nkv) * hd))
    _check(out, "out", torch.bfloat16, (B, nq * hd))
    pages = kv.k.shape[0]
    _check(kv.k, "key pages", torch.bfloat16, (pages, nkv, 64, hd))
    _check(kv.v, "value pages", torch.bfloat16, (pages, nkv, hd, 64))
    _check(kv.page_table, "page_table", torch.int32, (None, None))
    _check(meta.slots, "slots", torch.int32, (B,))
    _check(meta.context_lens, "context_lens", torch.int32, (B,))
    if not decode_fusable(meta, kv, nq, nkv, hd, hd if cos is not None else 0, torch.bfloat16):
        raise BackendError(f"fused decode attention refuses head_dim {hd} with {nq}/{nkv} heads in this step")
    for w, name in ((q_norm_w, "q_norm"), (k_norm_w, "k_norm")):
        if w is not None:
            _check(w, name, torch.float32, (hd,))
    if (cos is None) != (sin is None):
        raise BackendError("cos and sin tables come together")
    if cos is not None:
        _check(cos, "cos", torch.float32, (None, hd // 2))
        _check(sin, "sin", torch.float32, tuple(cos.shape))
        if meta.max_position >= cos.shape[0]:
            raise BackendError(f"position {meta.max_position} beyond the rotation table ({cos.shape[0]} rows)")
    window = int(window or 0)
    listed = _decode_ranges(meta, nkv, window)
    if listed:
        (splits, ranges), per = listed, 1
        po, pml = _partial_buffers(scratch, qkv.device, nq, splits, hd)
    else:
        (splits, per), ranges = _decode_split(meta, nkv, window), None
        po, pml = _partial_buffers(scratch, qkv.device, B * nq, splits, hd)
    n_slices, src, stride = qkv_slices if qkv_slices is not None else (1, qkv.data_ptr(), 0)
    if n_slices > 1 and (n_slices not in DEFERRED_SLICES or hd != 128 or stride < qkv.numel()):
        raise BackendError(f"fused decode attention does not add up {n_slices} slices of the projection")
    lib.call("attention_mfma", "hb_attn_decode_mfma", None, kv.k.data_ptr(), kv.v.data_ptr(), out.data_ptr(),
             po.data_ptr(), pml.data_ptr(), meta.context_lens.data_ptr(), meta.slots.data_ptr(),
             kv.page_table.data_ptr(), kv.page_table.shape[1], kv.page_size, B, nq, nkv, hd, float(scale),
             window, splits, per, src, None if q_norm_w is None else q_norm_w.data_ptr(),
             None if k_norm_w is None else k_norm_w.data_ptr(), None if cos is None else cos.data_ptr(),
             None if sin is None else sin.data_ptr(), float(eps), 1, n_slices, stride,
             None if ranges is None else ranges.data_ptr(), _stream())


DEFERRED_SLICES = (2, 4, 8)     # numbers of slices of the projection that the decode kernel adds up itself


def attention(q, meta, kv, out, nq, nkv, hd, scale, window, tile_height=None, scratch=None):
    """Causal (and windowed) attention of the step's tokens over their slots' pages.
    One token a sequence: the split decode kernel; otherwise one of the two tiled prompt kernels
    (tile_height 32 or 64 asks for one by name; None: the host's choice, see _prefill_tile_height)."""
    T = q.shape[0]
    _check(q, "q", torch.bfloat16, (T, nq * hd))
    _check(out, "out", torch.bfloat16, (T, nq * hd))
    pages = kv.k.shape[0]
    _check(kv.k, "key pages", torch.bfloat16, (pages, nkv, 64, hd))
    _check(kv.v, "value pages", torch.bfloat16, (pages, nkv, hd, 64))
    _check(kv.page_table, "page_table", torch.int32, (None, None))
    _check(meta.slots, "slots", torch.int32, (meta.num_seqs,))
    if not attention_supported(q, kv, nq, nkv, hd):
        raise BackendError(f"attention_mfma refuses head_dim {hd} with {nq}/{nkv} heads")
    window = int(window or 0)
    if meta.max_new == 1:
        if T != meta.num_seqs:
            raise BackendError("decode attention needs one token for each sequence")
        _check(meta.context_lens, "context_lens", torch.int32, (T,))
        listed = _decode_ranges(meta, nkv, window)
        if listed:
            (splits, ranges), per = listed, 1
            po, pml = _partial_buffers(scratch, q.device, nq, splits, hd)
        else:
            (splits, per), ranges = _decode_split(meta, nkv, window), None
            po, pml = _partial_buffers(scratch, q.device, T * nq, splits, hd)
        lib.call("attention_mfma", "hb_attn_decode_mfma", q.data_ptr(), kv.k.data_ptr(), kv.v.data_ptr(),
                 out.data_ptr(), po.data_ptr(), pml.data_ptr(), meta.context_lens.data_ptr(),
                 meta.slots.data_ptr(), kv.page_table.data_ptr(), kv.page_table.shape[1], kv.page_size,
                 T, nq, nkv, hd, float(scale), window, splits, per, None, None, None, None, None, 0.0, 0, 1, 0,
                 None if ranges is None else ranges.data_ptr(), _stream())
        return
    _check(meta.positions, "positions", torch.int32, (T,))
    height = tile_height or _prefill_tile_height(meta, nkv, nq // nkv)
    if height not in (32, 64):
        raise BackendError("prompt attention has tiles of 32 or of 64 tokens")
    tile_seq, tile_row0, tile_rows, n_tiles = _prefill_tiles(meta, height)
    lib.call("attention_mfma", "hb_attn_prefill_mfma", q.data_ptr(), kv.k.data_ptr(), kv.v.data_ptr(),
             out.data_ptr(), tile_seq.data_ptr(), tile_row0.data_ptr(), tile_rows.data_ptr(), n_tiles,
             meta.positions.data_ptr(), meta.slots.data_ptr(), kv.page_table.data_ptr(),
             kv.page_table.shape[1], kv.page_size, nq, nkv, hd, float(scale), window, height, _stream())
