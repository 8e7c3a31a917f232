"""The choice of kernel for a matrix product is made on the host: its invariants are checked
here without a GPU, over a grid of sizes (the library is compiled if it is not there yet)."""
import itertools

import pytest

from herbert_rs_amd.kernels import lib

EPI_STORE, EPI_ADD, EPI_SWIGLU = 0, 1, 2
TILES = {112: (128, 32), 124: (128, 64), 184: (256, 64), 122: (128, 128), 142: (256, 128), 188: (256, 256), 123: (128, 128),
         168: (192, 256), 164: (96, 64), 186: (256, 192)}


@pytest.fixture(scope="module")
def plan():
    from herbert_rs_amd.kernels import mfma  # noqa: F401  (registers the signatures)
    fn = lib.load("gemm_mfma").hb_gemm_mfma_plan

    def ask(M, N, K, epi=EPI_STORE, normed=False, emit=False, scaled=False, workspace=1 << 24, deferred=False):
        return fn(M, N, K, epi, int(normed), int(emit), int(scaled), workspace, int(deferred))
    return ask


ROWS = [1, 2, 7, 8, 16, 17, 32, 33, 64, 65, 100, 256, 700, 1024, 2048, 5000]
WIDTHS = [64, 1024, 2048, 4096, 5120, 6144, 12288, 24576, 151936]
DEPTHS = [64, 128, 512, 2048, 2112, 4096, 12288, 25600]


def test_every_plan_is_a_kernel_that_takes_the_product(plan):
    for M, N, K in itertools.product(ROWS, WIDTHS, DEPTHS):
        for epi in (EPI_STORE, EPI_ADD, EPI_SWIGLU):
            p = plan(M, N, K, epi)
            assert p >= 0, (M, N, K, epi)
            if p == 0:
                assert M <= 16
                continue
            tile, slices = p % 1000, max(1, p // 1000)
            assert tile in TILES and (tile != 112 or M <= 32), (M, N, K, p)
            assert tile not in (168, 164) or (epi == EPI_SWIGLU and slices == 1), (M, N, K, p)
            assert tile != 164 or 32 < M <= 64, (M, N, K, p)
            steps = K // 64
            if slices > 1:
                per = -(-steps // slices)
                assert per * (slices - 1) < steps, (M, N, K, p)            # no slice of K is empty
                assert steps // slices >= 4 and slices * M * N <= 1 << 24, (M, N, K, p)
                assert slices in (2, 4, 8, 16)


def test_without_a_workspace_k_is_never_cut(plan):
    for M, N, K in itertools.product(ROWS, WIDTHS, DEPTHS):
        assert plan(M, N, K, EPI_ADD, workspace=0) < 1000


def test_k_in_steps_of_32_only_goes_to_the_kernel_built_for_it(plan):
    for M in (1, 16, 17, 64, 300):
        p = plan(M, 4096, 4096 + 32)
        assert p == (0 if M <= 16 else 123)


def test_a_norm_is_left_behind_by_the_few_row_kernel_or_by_the_kernel_that_adds_slices(plan):
    for M, N, K in itertools.product([1, 8, 16, 17, 40, 64, 128, 512], [192, 2048, 4096, 5120, 8192], [512, 4096, 25600]):
        p = plan(M, N, K, EPI_ADD, emit=True)
        if M <= 16:
            assert p == 0 or p >= 2000, (M, N, K, p)
        else:
            assert p >= 2000 or p == -1, (M, N, K, p)          # -1: nothing fits; the caller then norms by itself
            if M <= 64:
                assert p >= 2000, (M, N, K, p)
    assert plan(40, 8196, 4096, EPI_ADD, emit=True) == -1      # rows too wide for the adding kernel
    assert plan(40, 4096, 4096, EPI_ADD, emit=True, workspace=0) == -1


def test_a_handed_on_norm_is_finished_by_the_few_row_kernel_or_the_128x32_tile(plan):
    for M, N, K in itertools.product([1, 8, 16], [1024, 6144, 24576, 51200], [1024, 4096, 5120]):
        for epi in (EPI_STORE, EPI_SWIGLU):
            p = plan(M, N, K, epi, scaled=True)
            assert p == 0 or p % 1000 == 112, (M, N, K, epi, p)


def test_slices_left_to_the_next_kernel_are_2_4_or_8(plan):
    for M, N, K in itertools.product([1, 8, 16, 40, 100, 256, 700], [1024, 4096, 6144, 10240], [2048, 4096, 8192, 25600]):
        p = plan(M, N, K, deferred=True)
        assert p // 1000 in (0, 2, 4, 8), (M, N, K, p)


def test_known_choices(plan):
    """A few choices that measurements decided: decoding 8 rows of the 8B shape, its prompt of 2048."""
    assert plan(8, 4096, 4096, EPI_ADD, emit=True) == 0                # o: the few-row kernel
    assert plan(8, 24576, 4096, EPI_SWIGLU, scaled=True) == 112        # gate/up: 128 x 32 tiles, no slices
    assert plan(8, 5120, 25600, EPI_ADD, emit=True) >= 2000            # hidden 5120: 320 workgroups would not spread
    assert plan(2048, 24576, 4096, EPI_SWIGLU) == 188
    assert plan(2048, 4096, 12288, EPI_ADD) == 142
    assert plan(64, 24576, 4096, EPI_SWIGLU) == 164                    # 256 tiles of 96 columns, not 192 of 128
    assert plan(32, 24576, 4096, EPI_SWIGLU) == 112 and plan(64, 51200, 5120, EPI_SWIGLU) % 1000 in (124, 184)


def test_rows_just_past_whole_tiles_are_cut_off_as_a_product_of_their_own():
    """A product whose rows end a little past a whole number of large tiles would pay a round of
    tiles for them: it is cut in two along its rows where the estimates say so, never where the
    rows fill their tiles, and never for few rows."""
    from herbert_rs_amd.kernels import mfma  # noqa: F401
    split = lib.load("gemm_mfma").hb_gemm_mfma_split
    W = 1 << 26
    H, I = 4096, 12288
    for M in (2049, 2064, 2112):
        assert split(M, 2 * I, H, EPI_SWIGLU, W) == 2048 and split(M, H, I, EPI_ADD, W) == 2048, M
    assert split(2049, 2 * I, H, EPI_SWIGLU, 0) == 2048           # (a rest of few rows needs no room for K slices)
    for M in (1, 16, 64, 128, 1024, 2048, 2304, 4096):
        for N, K, epi in ((2 * I, H, EPI_SWIGLU), (H, I, EPI_ADD), (H, H, EPI_ADD), (6144, H, EPI_STORE)):
            assert split(M, N, K, epi, W) == 0, (M, N, K)
    for M, N, K in itertools.product([130, 257, 300, 513, 700, 1025, 1500, 3000, 5000], WIDTHS, [512, 2048, 4096, 12288]):
        for epi in (EPI_STORE, EPI_ADD, EPI_SWIGLU):
            for ws in (0, W):
                rows = split(M, N, K, epi, ws)
                assert rows == 0 or (0 < rows < M and rows % 128 == 0 and M - rows < 256), (M, N, K, epi, rows)


def test_decode_attention_ranges_by_how_evenly_the_waves_sit():
    """One range a (sequence, kv head) from 512 of them on, unless the waves would sit unevenly on
    the CUs (three on some where most have two, or a second round that is a quarter full): then
    eight shorter ranges; below, as many ranges as fill one round of 1,024 waves."""
    from herbert_rs_amd.kernels import mfma

    class Meta:
        def __init__(self, seqs, tokens):
            self.num_seqs, self.context_bucket = seqs, tokens
    split = lambda b, t=4096, nkv=8, window=0: mfma._decode_split(Meta(b, t), nkv, window)
    assert split(1) == (32, 2) and split(8) == (16, 4) and split(32) == (4, 16) and split(48) == (2, 32)
    for b in (64, 80, 96, 128, 200, 256):
        assert split(b) == (1, 64), b
    for b in (65, 72, 136, 160):
        assert split(b) == (8, 8), b
    assert split(65, 1024) == (4, 4) and split(65, 512) == (1, 8)
    assert split(65, 4096, window=100) == (1, 3)
    for b in range(1, 300, 7):
        for t in (64, 700, 4096, 32768):
            ranges, per = split(b, t)
            span = -(-t // 64)
            assert ranges >= 1 and per >= 1 and ranges * per >= span > (ranges - 1) * per, (b, t)


def test_decode_attention_takes_a_list_of_ranges_only_where_it_fits():
    """The list that deals the decode grid out over sequences of unequal lengths: for two sequences
    or more without a window, a round of waves or two items a sequence, up to the kernel's 1,024
    items; else equal shares."""
    import torch
    from herbert_rs_amd.engine.batch import StepEntry, pack, range_list
    from herbert_rs_amd.kernels import mfma

    def meta_of(contexts):
        return pack([StepEntry(i, [1], [0]) for i in range(len(contexts))], [c - 1 for c in contexts],
                    torch.device("cpu"))
    unequal = [9000] + [100] * 7
    items, listed = mfma._decode_ranges(meta_of(unequal), 8, 0)
    assert items == 128 and listed.tolist() == range_list(unequal, 128, 64).tolist()
    assert mfma._decode_ranges(meta_of(unequal), 2, 0)[0] == 512
    assert mfma._decode_ranges(meta_of(unequal), 1, 0)[0] == 1024           # the grid's z has no more
    assert mfma._decode_ranges(meta_of(unequal), 8, 70) is None             # a window
    assert mfma._decode_ranges(meta_of([9000] * 4 + [8000] * 4), 8, 0) is None      # lengths alike
    assert mfma._decode_ranges(meta_of([9000]), 8, 0) is None
    assert mfma._decode_ranges(meta_of([9000] + [100] * 64), 8, 0)[0] == 130   # two items a sequence
    assert mfma._decode_ranges(meta_of([9000] + [100] * 39), 16, 0)[0] == 80
    assert mfma._decode_ranges(meta_of([9000] + [100] * 31), 16, 0)[0] == 64
    assert mfma._decode_ranges(meta_of([9000] + [100] * 511), 8, 0)[0] == 1024
    assert mfma._decode_ranges(meta_of([9000] + [100] * 512), 8, 0) is None     # more items than the kernel takes
    half = [4000] * 40 + [200] * 40                             # holds 0.525 of 80 x 4000: level 1
    assert meta_of(half).unequal == 1 and meta_of(half[8:72]).unequal == 1
    assert mfma._decode_ranges(meta_of(half), 8, 0) is None     # more than a round of waves: from level 2 on
    assert mfma._decode_ranges(meta_of(half[8:72]), 8, 0)[0] == 128
    prompt = pack([StepEntry(0, [1, 2, 3], [2]), StepEntry(1, [4], [0])], [9000, 10], torch.device("cpu"))
    assert prompt.unequal and mfma._decode_ranges(prompt, 8, 0) is None     # not one token a sequence
