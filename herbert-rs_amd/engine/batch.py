"""The tokens of one step, packed over the sequences of the batch, with what kernels need
to find each token's sequence, position and pages.

The reference steps one sequence at a time (crates/backends/backend_common/src/generic_model.rs:131 prompts with a
start position, :524 one token); a batch of unequal sequences in one step has no counterpart
there. Its checks are kept: no empty sequence, ids below the vocabulary, positions below
max_position_embeddings (crates/backends/backend_common/src/generic_model.rs:139-152, 165-171, 531-537)."""
from dataclasses import dataclass
from typing import List

import numpy as np
import torch


@dataclass
class StepEntry:
    """One sequence's share of a step: its slot, its next tokens and the places among
    them whose logits are wanted."""
    slot: int
    tokens: List[int]
    want: List[int]


@dataclass
class BatchMeta:
    token_ids: torch.Tensor    # int32 [T]
    positions: torch.Tensor    # int32 [T]   absolute position of each token in its sequence
    seq_of: torch.Tensor       # int32 [T]   index of the token's sequence in this batch
    slots: torch.Tensor        # int32 [B]   slot of each sequence
    seq_starts: torch.Tensor   # int32 [B+1] first packed row of each sequence
    context_lens: torch.Tensor  # int32 [B]  positions held after this step
    want_rows: torch.Tensor    # int32 [R]   packed rows whose logits are wanted
    num_tokens: int
    num_seqs: int
    max_new: int               # most tokens any sequence brings
    max_context: int           # largest context length after this step
    max_position: int          # largest absolute position in the step
    host_starts: np.ndarray    # host copies, for kernels' grids
    host_context: np.ndarray
    derived: dict = None       # what kernels' host sides derive once a step (tile lists and the like)
    context_bucket: int = 0    # max_context rounded up (see bucket): sizes the decode kernels' grids
    unequal: int = 0           # how unequal the contexts' lengths are: 0 (alike), 1, 2 (see unequal_level)
    num_real: int = 0          # sequences that are no padding rows (0: all of them)
    static: object = None      # the StaticDecodeMeta whose buffers these are, if any

    def ranges_for(self, items, unit):
        """The list that cuts this step's contexts into at most `items` ranges of equally many whole
        units of `unit` positions (see range_list), as int32 [num_seqs + 2] on the GPU; None if a
        step with fixed buffers has no room for another list. A step with fixed buffers refills the
        lists it has handed out at every update whose sequences are `unequal`: ask only then."""
        key = ("ranges", int(items), int(unit))
        got = self.derived.get(key)
        if got is None:
            if self.static is not None:
                got = self.static.add_range_list(int(items), int(unit))
                if got is None:
                    return None
            else:
                got = torch.from_numpy(range_list(self.host_context, items, unit)).to(self.token_ids.device)
            self.derived[key] = got
        return got


def unequal_level(context):
    """How unequal the lengths of a step's sequences are, by what they hold together of what they
    would if all were as long as the longest: 0 above 0.55, 1 from there down, 2 from 0.45 down. A
    kernel that gives every sequence the same share of the GPU leaves much of it idle where this
    is not 0. (Measured on decode steps of the 8B shape: dealing the attention's grid out by a list
    takes 7 to 11 % off a step of 8 to 64 sequences at 0.34 to 0.51 and 23 to 54 % at 0.08 to
    0.18, nothing from 0.56 on, and adds 2 to 4 % where all are equal. 80 to 200 sequences, whose
    lists need more than one round of waves: 9 to 36 % off at 0.17 to 0.40, 60 % at 0.07, between
    9 % more and 7 % less at 0.5: these take the list from level 2 on.)"""
    context = np.asarray(context, dtype=np.int64)
    if len(context) < 2:
        return 0
    held, room = 20 * int(context.sum()), len(context) * int(context.max())
    return 2 if held <= 9 * room else 1 if held <= 11 * room else 0


def range_list(context, items, unit):
    """Cut B sequences of unequal lengths into ranges of equally many whole units (pages), at most
    `items` of them together (items > B): int32 [B + 2] with [0 .. B] the number of ranges of the
    sequences before each one and [B + 1] the units of a range, the fewest with which every
    sequence's ranges, rounded up, still fit. (They do at sum p / (items - B) units: sum ceil(p / per)
    < sum p / per + B <= items; and the number of ranges never grows with the units a range has.)"""
    context = np.asarray(context, dtype=np.int64)
    B = len(context)
    if items <= B:
        raise ValueError(f"{items} ranges cannot be dealt out to {B} sequences")
    units = np.maximum(1, -(-context // unit))
    total = int(units.sum())
    low, high = max(1, -(-total // items)), max(1, -(-total // (items - B)))      # high always fits
    while low < high:
        per = (low + high) // 2
        if int((-(-units // per)).sum()) <= items:
            high = per
        else:
            low = per + 1
    out = np.empty(B + 2, dtype=np.int32)
    out[0] = 0
    np.cumsum(-(-units // high), out=out[1:B + 1])
    out[B + 1] = high
    return out


CONTEXT_BUCKET = 256


def bucket(context):
    """The context rounded up to what sizes a decode kernel's grid (and names a captured graph):
    multiples of 256 up to 4,096 tokens, of 512 up to 8,192, of 1,024 up to 16,384 and so on, so that
    a sequence that grows long passes through 8 buckets for each doubling and a grid is never
    more than an eighth too large."""
    context, step = int(context), CONTEXT_BUCKET
    while context > 16 * step:
        step *= 2
    return (context + step - 1) // step * step


def pack(entries, start_lengths, device, staging=None):
    """Build the BatchMeta of a step. start_lengths[i] is what entry i's slot holds already."""
    B = len(entries)
    counts = [len(e.tokens) for e in entries]
    T = sum(counts)
    R = sum(len(e.want) for e in entries)
    starts = np.zeros(B + 1, dtype=np.int32)
    starts[1:] = np.cumsum(counts)
    total = 3 * T + B + (B + 1) + B + R
    host = np.empty(total, dtype=np.int32)
    tok = host[0:T]
    pos = host[T:2 * T]
    seq = host[2 * T:3 * T]
    o = 3 * T
    slots = host[o:o + B]
    o += B
    host[o:o + B + 1] = starts
    o += B + 1
    ctx = host[o:o + B]
    o += B
    want = host[o:o + R]
    w = 0
    for i, e in enumerate(entries):
        a, b = starts[i], starts[i + 1]
        tok[a:b] = e.tokens
        pos[a:b] = np.arange(start_lengths[i], start_lengths[i] + counts[i], dtype=np.int32)
        seq[a:b] = i
        slots[i] = e.slot
        ctx[i] = start_lengths[i] + counts[i]
        for j in e.want:
            want[w] = a + j
            w += 1
    dev = torch.from_numpy(host).to(device)
    o = 3 * T
    return BatchMeta(
        token_ids=dev[0:T], positions=dev[T:2 * T], seq_of=dev[2 * T:3 * T],
        slots=dev[o:o + B], seq_starts=dev[o + B:o + 2 * B + 1],
        context_lens=dev[o + 2 * B + 1:o + 3 * B + 1], want_rows=dev[o + 3 * B + 1:o + 3 * B + 1 + R],
        num_tokens=T, num_seqs=B, max_new=max(counts), max_context=int(ctx.max()),
        max_position=int(pos.max()), host_starts=starts.copy(), host_context=ctx.copy(), derived={},
        context_bucket=bucket(int(ctx.max())), unequal=unequal_level(ctx))


def decode_batch_bucket(sequences):
    """The batch size that a decode step of `sequences` sequences runs at: 1, 2, 3, 4, 6, 8, then four
    sizes for every doubling up to 64 (10, 12, 14, 16, 20, 24, 28, 32, 40, ...) and eight beyond (72,
    80, 88, ...), the rows beyond the sequences being padding. Every size is a shape that the host
    has to walk through once and record; a batch whose sequences end one after another then meets
    ten shapes on its way down from 16 instead of sixteen. A padding row is not free where a
    kernel's time goes with its rows (the few-row product reads its activations once a workgroup:
    about 2 % a row; beyond 64 sequences every eighth more is another wave on some CUs of the
    attention), so the sizes stay within an eighth to a quarter of the sequences (measured on the
    1.7B shape, 16 sequences that end 14 tokens apart: rounding up to powers of two took 3 % more
    time for the 250 steps than exact sizes)."""
    n = max(1, int(sequences))
    if n <= 4:
        return n
    top = 1 << (n - 1).bit_length()          # the power of two at or above n
    step = 2 if n <= 8 else top // 8 if n <= 64 else top // 16
    return -(-n // step) * step


class StaticDecodeMeta:
    """The metadata of a step of B sequences with one token each, every logit wanted, in buffers
    that stay where they are: a captured graph reads them, `update` refills them. A step may
    bring fewer sequences than B: the rows left over are padding, each a sequence of one token (id
    0, position 0) in the cache's padding slot; what they compute is thrown away, and no other
    row's result depends on them."""

    RANGE_LISTS = 4      # lists of ranges (BatchMeta.ranges_for) that the buffers have room for

    def __init__(self, batch_size, device, pad_slot=0):
        B = self.batch_size = batch_size
        self.pad_slot = int(pad_slot)
        size = 7 * B + 1 + self.RANGE_LISTS * (B + 2)
        self.host = torch.zeros(size, dtype=torch.int32, pin_memory=torch.device(device).type == "cuda")
        self.copied = None       # event after the last copy out of `host`
        self.dev = torch.zeros(size, dtype=torch.int32, device=device)
        self.range_lists = []    # (items, unit) of the lists handed out, in the order of their places
        h = self.host_array = self.host.numpy()
        h[2 * B:3 * B] = np.arange(B)            # seq_of
        h[4 * B:5 * B + 1] = np.arange(B + 1)    # seq_starts
        h[6 * B + 1:7 * B + 1] = np.arange(B)    # want_rows
        d = self.dev
        self.meta = BatchMeta(
            token_ids=d[0:B], positions=d[B:2 * B], seq_of=d[2 * B:3 * B], slots=d[3 * B:4 * B],
            seq_starts=d[4 * B:5 * B + 1], context_lens=d[5 * B + 1:6 * B + 1],
            want_rows=d[6 * B + 1:7 * B + 1], num_tokens=B, num_seqs=B, max_new=1, max_context=0,
            max_position=0, host_starts=np.arange(B + 1, dtype=np.int32),
            host_context=np.zeros(B, dtype=np.int32), derived={}, context_bucket=0, static=self)

    def _range_place(self, i):
        first = 7 * self.batch_size + 1 + i * (self.batch_size + 2)
        return slice(first, first + self.batch_size + 2)

    def add_range_list(self, items, unit):
        """A place in the buffers for the list (items, unit), filled for the step at hand and from
        now on at every update; None if all places are taken. Not under graph capture: the list is
        copied to the GPU here, so a step's first, eager run has to be the one that asks."""
        if len(self.range_lists) == self.RANGE_LISTS:
            return None
        if self.dev.is_cuda and torch.cuda.is_current_stream_capturing():
            from ..errors import NeedsEagerStep
            raise NeedsEagerStep("a list of ranges is first asked for while a graph is recorded")
        place = self._range_place(len(self.range_lists))
        self.range_lists.append((items, unit))
        self.host_array[place] = range_list(self.meta.host_context, items, unit)
        self.dev[place].copy_(self.host[place])
        return self.dev[place]

    def update(self, entries, start_lengths):
        B, n = self.batch_size, len(entries)
        if n > B:
            raise ValueError(f"{n} sequences do not fit a step of {B}")
        if self.copied is not None:
            self.copied.synchronize()        # the pinned buffer is free to be written again
        h = self.host_array
        h[0:n] = [e.tokens[0] for e in entries]
        h[B:B + n] = start_lengths
        h[3 * B:3 * B + n] = [e.slot for e in entries]
        if n < B:                            # padding rows
            h[n:B] = 0
            h[B + n:2 * B] = 0
            h[3 * B + n:4 * B] = self.pad_slot
        context = h[5 * B + 1:6 * B + 1]
        np.add(h[B:2 * B], 1, out=context)
        unequal = unequal_level(context[:n])         # of the sequences themselves
        if unequal:                     # nobody reads the lists of a step whose sequences are alike
            for i, (items, unit) in enumerate(self.range_lists):
                h[self._range_place(i)] = range_list(context, items, unit)
        self.dev.copy_(self.host, non_blocking=True)
        if self.dev.is_cuda:
            if self.copied is None:
                self.copied = torch.cuda.Event()
            self.copied.record()
        m = self.meta
        m.host_context = context.copy()
        m.max_context = int(max(start_lengths)) + 1
        m.max_position = m.max_context - 1
        m.context_bucket = bucket(m.max_context)
        m.unequal = unequal
        m.num_real = n
        return m
