"""Choosing tokens on the GPU from float32 logits.

temperature 0: the first index of the largest value (crates/core/src/sampler.rs:244-254).
Otherwise the reference's algorithm (sampler.rs:72-145): divide by the temperature, keep the
top_k largest, softmax, keep the shortest prefix by descending probability whose sum reaches
top_p, renormalise, walk the running sum until it exceeds the draw. Where the reference
leaves the order of candidates open, it is value descending, index ascending among equals.
"""
import torch

from ..errors import RequestError
from ..kernels import ops
from . import xorshift
from .think import ThinkBudget


def _signed64(v):
    return v - (1 << 64) if v >= (1 << 63) else v


class PendingTokens:
    """Tokens that have been chosen on the GPU and are on their way to the host: `device` (int32
    [rows]) can feed the next step at once, `Sampler.read` waits for the copy and gives the list."""

    def __init__(self, device, host, event):
        self.device, self.host, self.event = device, host, event


class Sampler:
    """One generator stream per sequence, kept on the GPU and advanced by the kernel."""

    def __init__(self, params, num_sequences, vocab_size, device):
        params.validate()
        self.params = params
        self.device = device
        self.vocab_size = vocab_size
        seed = params.seed if params.seed is not None else xorshift.clock_seed()
        states = [_signed64(xorshift.sequence_seed(seed, i)) for i in range(num_sequences)]
        self.states = torch.tensor(states, dtype=torch.int64, device=device)
        self._scratch = None
        self._sifted = None
        self._nucleus = None
        self._sums = None
        self._argmax_scratch = None
        self._host_ring = []            # pinned buffers that tokens on their way to the host land in
        self._host_next = 0
        self._index = None
        self._row_indices = {}          # (rows of a choice, the rows taken) -> their index on the GPU
        # a cap on think blocks: one counter a sequence, fed with every token chosen for it
        self.think = None
        if params.think_budget > 0:
            self.think = [ThinkBudget(params.think_budget, params.think_tokens) for _ in range(num_sequences)]

    def new_turn(self):
        """A conversation's next turn: its think blocks begin closed (crates/cli/src/chat.rs:1119);
        the generator streams go on."""
        for t in self.think or ():
            t.reset()

    def save_streams(self):
        """A copy of every sequence's generator state as it is at this point of the stream (no
        waiting): for a caller that may have to take a draw back (`restore_stream`)."""
        return self.states.clone()

    def restore_stream(self, sequence, saved):
        """Put sequence `sequence`'s generator state back to what `saved` (a `save_streams`) holds."""
        self.states[sequence:sequence + 1].copy_(saved[sequence:sequence + 1])

    def _sifted_for(self, rows):
        """Buffers for the candidates that a block a chunk sifts out of a long row (top-k up to 1024)."""
        p = self.params
        if not (0 < p.top_k < self.vocab_size and p.top_k <= 1024) or self.vocab_size <= 2 * ops.SAMPLE_CHUNK:
            return None
        need = rows * (-(-self.vocab_size // ops.SAMPLE_CHUNK)) * p.top_k
        if self._sifted is None or self._sifted[0].numel() < need:
            self._sifted = (torch.empty(need, dtype=torch.int32, device=self.device),
                            torch.empty(need, dtype=torch.int32, device=self.device))
        return self._sifted

    def _scratch_for(self, rows):
        p = self.params
        if 0 < p.top_k < self.vocab_size and p.top_k <= 1024:
            return None
        p2 = 1
        while p2 < self.vocab_size:
            p2 <<= 1
        if self._scratch is None or self._scratch[0].shape[0] < rows:
            self._scratch = (torch.empty((rows, p2), dtype=torch.int32, device=self.device),
                             torch.empty((rows, p2), dtype=torch.int32, device=self.device))
        return self._scratch

    def choose(self, logits, sequence_indices):
        """Token for each row of `logits`; row r belongs to sequence sequence_indices[r]. Where a
        sequence's think block has used its budget, the row is first left with the one token that
        may follow (the logits are changed in place), then chosen from as every row is: a draw
        is taken for it as for any other."""
        if self.think is None:
            return self._choose(logits, sequence_indices)
        sequence_indices = list(sequence_indices)
        forced = [(r, self.think[s].forced()) for r, s in enumerate(sequence_indices)]
        forced = [(r, t) for r, t in forced if t is not None]
        if forced:
            ops.force_tokens(logits, [r for r, _ in forced], [t for _, t in forced])
        tokens = self._choose(logits, sequence_indices)
        for s, t in zip(sequence_indices, tokens):
            self.think[s].track(t)
        return tokens

    def _needs_host(self, vocab):
        """True where the choice of a token takes a decision of the host in between: a think
        budget (the forced token depends on the one before), top-p without top-k (rows that the
        quick kernel leaves go the general way)."""
        p = self.params
        return self.think is not None or (not p.greedy and not 0 < p.top_k < vocab and p.top_p < 1.0
                                          and vocab > ops.NUCLEUS_CANDIDATES)

    @property
    def can_run_ahead(self):
        """Whether `choose_ahead` may be used: the tokens then stay on the GPU, where the next
        step can take them from, and the host reads them later."""
        return not self._needs_host(self.vocab_size)

    def choose_ahead(self, logits, sequence_indices):
        """Like `choose`, without waiting: the kernels are put on the stream, the tokens are copied
        to the host behind them, and a PendingTokens is returned at once."""
        if self._needs_host(logits.shape[1]):
            raise RequestError("these sampling parameters need the host between two choices")
        out = self._on_device(logits, sequence_indices)
        rows = out.shape[0]
        ring = self._host_ring
        if not ring or ring[0].shape[0] < rows:
            ring[:] = [torch.empty(max(rows, 64), dtype=torch.int32, pin_memory=True) for _ in range(4)]
        host = ring[self._host_next % len(ring)][:rows]
        self._host_next += 1
        host.copy_(out, non_blocking=True)
        event = torch.cuda.Event()
        event.record()
        return PendingTokens(out, host, event)

    @staticmethod
    def read(pending):
        """The tokens of a `choose_ahead`, once they have arrived."""
        pending.event.synchronize()
        return pending.host.tolist()

    def rows_of(self, pending, rows):
        """The device tokens of some rows of a `choose_ahead`, in the given order. The index of a
        choice of rows is kept: a batch that shrinks asks for the same rows step after step, and
        making the index anew would wait for a copy from the host each time."""
        rows = tuple(rows)
        if rows == tuple(range(pending.device.shape[0])):
            return pending.device
        key = (pending.device.shape[0], rows)
        index = self._row_indices.get(key)
        if index is None:
            if len(self._row_indices) >= 256:
                self._row_indices.clear()
            host = torch.tensor(rows, dtype=torch.long).pin_memory() if self.device.type == "cuda" \
                else torch.tensor(rows, dtype=torch.long)
            index = self._row_indices[key] = host.to(self.device, non_blocking=True)
        return pending.device[index]

    def _index_of(self, sequence_indices):
        """The rows' sequences as a tensor on the GPU; the one of the step before is kept, since a
        batch keeps its sequences for many steps (and a copy from the host would wait for the GPU)."""
        key = tuple(sequence_indices)
        if self._index is None or self._index[0] != key:
            self._index = (key, torch.tensor(key, dtype=torch.int32, device=self.device))
        return self._index[1]

    def _on_device(self, logits, sequence_indices):
        """The choice for every row as an int32 tensor on the GPU; only where no decision of the
        host is needed in between."""
        rows = logits.shape[0]
        out = torch.empty(rows, dtype=torch.int32, device=self.device)
        p = self.params
        if p.greedy:
            if self._argmax_scratch is None or self._argmax_scratch[0].shape[0] < rows:
                self._argmax_scratch = ops.argmax_scratch(rows, self.device)
            ops.argmax(logits, out, self._argmax_scratch)
            return out
        index = self._index_of(sequence_indices)
        vocab = logits.shape[1]
        if not 0 < p.top_k < vocab and p.top_p >= 1.0 and vocab > ops.SAMPLE_CHUNK:
            # the whole row, no cut: nothing is sorted, the chunks of a long row are added up side by side
            need = rows * (-(-vocab // ops.SAMPLE_CHUNK)) * 2
            if self._sums is None or self._sums.numel() < need:
                self._sums = torch.empty(need, dtype=torch.float32, device=self.device)
            ops.sample_all(logits, p.temperature, self.states, index, out, self._sums)
            return out
        ops.sample(logits, p.temperature, p.top_k, p.top_p,
                   self.states, index, out, self._scratch_for(rows), self._sifted_for(rows))
        return out

    def _choose(self, logits, sequence_indices):
        p = self.params
        vocab = logits.shape[1]
        if not p.greedy and not 0 < p.top_k < vocab and p.top_p < 1.0 and vocab > ops.NUCLEUS_CANDIDATES:
            index = torch.tensor(list(sequence_indices), dtype=torch.int32, device=self.device)
            out = torch.empty(logits.shape[0], dtype=torch.int32, device=self.device)
            return self._top_p_only(logits, index, out)
        return self._on_device(logits, sequence_indices).tolist()

    def _top_p_only(self, logits, index, out):
        """Top-p without top-k: first among each row's 1024 largest logits, where the prefix that
        reaches top_p nearly always ends (no sort of the whole vocabulary); the rows where it does
        not (flat distributions) then go the general way, with the same draw."""
        rows, p = logits.shape[0], self.params
        if self._nucleus is None or self._nucleus[2].numel() < rows * (-(-logits.shape[1] // ops.SAMPLE_CHUNK)) * 2:
            self._nucleus = ops.nucleus_buffers(rows, logits.shape[1], self.device)
        ops.sample_nucleus(logits, p.temperature, p.top_p, self.states, index, out, self._nucleus)
        tokens = out.tolist()
        rest = [r for r, t in enumerate(tokens) if t < 0]
        if rest:
            at = torch.tensor(rest, dtype=torch.long, device=self.device)
            sub_out = torch.empty(len(rest), dtype=torch.int32, device=self.device)
            ops.sample(logits[at].contiguous(), p.temperature, p.top_k, p.top_p, self.states,
                       index[at].contiguous(), sub_out, self._scratch_for(len(rest)), None)
            for r, t in zip(rest, sub_out.tolist()):
                tokens[r] = t
        return tokens
