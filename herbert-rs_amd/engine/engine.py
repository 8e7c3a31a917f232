"""The engine: a model on the GPU, its cache, and the one step function.

`step` takes a batch of sequences with unequal numbers of new tokens (whole
prompts in a batch's first step, one token each afterwards), runs exactly
those tokens against the cache as one packed batch and returns the float32
logits at the wanted places. The reference's counterparts are per sequence:
prefill_with_token, decode_step and verify_draft_tokens
(crates/backends/backend_common/src/generic_model.rs:131,524,737); its error
cases are kept: empty input (:139-152), token id >= vocab (:165-171), position
beyond max_position_embeddings (:531-537).
"""
from collections import OrderedDict

import numpy as np
import torch

from ..cache import Cache
from ..config import load_config
from ..errors import BackendError, ModelLoadError, NeedsEagerStep, RequestError
from ..parts import Runtime
from ..weights import read_tensor, read_tensors

from . import batch as batching
from .batch import StaticDecodeMeta, StepEntry, decode_batch_bucket
from .model import Model

_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16,
           torch.float32: torch.float32, torch.bfloat16: torch.bfloat16}


class _DecodeState:
    """What the decode steps of one batch size share: the fixed metadata buffers and the rows of
    the engine's logits buffer that every graph of this batch size writes to."""

    def __init__(self, static, logits):
        self.static = static
        self.logits = logits


# Captured graphs kept at any time, over all batch sizes and context buckets; the least recently
# replayed one is dropped for a new one. A graph holds no logits of its own and no scratch (the
# parts' buffers are the runtime's), so a graph costs its kernel arguments only; the cap bounds
# what a long run over many batch sizes and contexts accumulates. A batch whose sequences end one
# after another passes through the sizes of the ladder below its first (batch.decode_batch_bucket),
# and each (size, context bucket) is a graph: the cap leaves room for many such batches' graphs, so
# that the next batch finds them.
MAX_GRAPHS = 192
# Decode steps write their logits into the first rows of one buffer [rows, vocab] float32 that the
# engine keeps (`step` hands out a copy of them unless it is asked for the rows themselves). The
# buffer starts with this many rows (39 MB for a vocabulary of 151,936) or as many as the cache's
# slots need, if fewer; a larger batch makes a larger one (twice the rows, or what the batch needs)
# and every graph, which holds the old one's address, is dropped.
SHARED_LOGITS_ROWS = 64
# Batch sizes whose fixed metadata buffers are kept; the least recently used goes, with its graphs.
MAX_DECODE_BATCH_SIZES = 96


def require_gpu():
    if not torch.cuda.is_available():
        raise BackendError("no GPU: this library runs on a gfx950 GPU only and has no other path")
    return torch.device("cuda", torch.cuda.current_device())


class Engine:
    def __init__(self, config, spec, tensors, dtype="bfloat16", max_tokens=4096, max_slots=None,
                 device=None, use_graphs=True):
        """tensors: {name: tensor} for the model's needs (any device)."""
        if dtype not in _DTYPES:
            raise BackendError(f"dtype must be float32 or bfloat16, got {dtype!r}")
        self.device = torch.device(device) if device is not None else require_gpu()
        self.config = config
        self.spec = spec
        self.rt = Runtime(_DTYPES[dtype], self.device)
        self.model = Model(spec)
        self.model.load(tensors, self.rt)
        self._check_cache_fits(max_tokens, max_slots)
        self.cache = Cache(self.model.cache_needs(), max_tokens, spec.max_positions, self.rt.dtype,
                           self.device, max_slots)
        self.steps_run = 0
        # Steps in which every sequence brings one token and wants its logits keep their metadata in
        # fixed buffers and run at a batch size of a ladder (see _decode_step), as graphs if asked
        # for: only for models whose parts do nothing but enqueue GPU work.
        self.static_decode = self.model.graph_safe
        self.use_graphs = bool(use_graphs) and self.model.graph_safe
        self._decode = OrderedDict()    # batch size -> _DecodeState, least recently used first
        self._graphs = OrderedDict()    # (batch size, context bucket, unequal) -> graph, least recently used first
        self._shared_logits = None      # [rows, vocab], made by the first decode step, grown by a larger batch
        self._capture_stream = None     # the stream that graphs are captured on
        self._sized_rows = 0            # the largest decode step that has run outside a graph: buffers for it exist
        self.graphs_captured = 0
        self.ignored_tensors = []       # stored tensors that the model did not ask for
        self._tensor_source = None      # how get_tensor finds a tensor again: set by the constructors below

    def _check_cache_fits(self, max_tokens, max_slots=None):
        """Refuse a cache that the GPU's free memory cannot hold, in the library's own words,
        before the allocator fails on it: keys and values by pages, fixed-size state by slots."""
        if self.device.type != "cuda":
            return
        needed = Cache.bytes_needed(self.model.cache_needs(), max_tokens, self.rt.dtype, max_slots)
        free, _ = torch.cuda.mem_get_info(self.device)
        if needed > free:
            from ..errors import CacheError
            raise CacheError(f"a cache of {max_tokens} tokens needs {needed / 2**30:.1f} GiB of keys, values "
                             f"and per-sequence state, {free / 2**30:.1f} GiB of GPU memory are free")

    # ---- construction
    @classmethod
    def from_folder(cls, folder, dtype="bfloat16", max_tokens=4096, max_slots=None, device=None,
                    use_graphs=True):
        """The engine of the model in `folder` (config.json + safetensors)."""
        arch, config = load_config(folder)
        spec = arch.build_spec(config)
        needs = Model(spec).tensor_needs()
        ignored = []
        tensors = read_tensors(folder, needs, name_map=arch.name_map, ignored=ignored)
        engine = cls(config, spec, tensors, dtype, max_tokens, max_slots, device, use_graphs)
        engine._tensor_source = lambda name: read_tensor(folder, name, needs, arch.name_map)
        engine.ignored_tensors = ignored
        engine.architecture = arch
        return engine

    @classmethod
    def from_config(cls, config, architecture=None, seed=0, dtype="bfloat16", weight_dtype=None,
                    std=0.02, norm_std=0.0, max_tokens=4096, max_slots=None, device=None, use_graphs=True):
        """An engine with seeded random weights drawn on the GPU (no files)."""
        from ..config.registry import resolve_architecture
        from ..weights import random_tensors
        arch = architecture or resolve_architecture(config.to_dict())
        spec = arch.build_spec(config)
        dev = torch.device(device) if device is not None else require_gpu()
        needs = Model(spec).tensor_needs()
        tensors = random_tensors(needs, seed, weight_dtype or dtype, std, norm_std, device=str(dev))
        engine = cls(config, spec, tensors, dtype, max_tokens, max_slots, dev, use_graphs)

        def again(name):
            if name not in needs:
                raise ModelLoadError(f"the model has no tensor {name!r}; it has: " + ", ".join(sorted(needs)))
            return random_tensors({name: needs[name]}, seed, weight_dtype or dtype, std, norm_std,
                                  device=str(dev))[name].cpu()
        engine._tensor_source = again
        engine.architecture = arch
        return engine

    def get_tensor(self, name):
        """The weight tensor `name` (the checkpoint's own name) as it is stored, on the CPU. The
        parts keep their weights in the order their kernels want; this reads the tensor again from
        where the engine's weights came from."""
        if self._tensor_source is None:
            raise ModelLoadError("this engine was built from tensors in memory; it cannot read them again")
        return self._tensor_source(name)

    # ---- slots
    def alloc_slot(self):
        return self.cache.alloc_slot()

    def free_slot(self, slot):
        self.cache.free_slot(slot)

    def truncate(self, slot, length):
        """Roll a sequence back to its first `length` positions; the next step's tokens go on from
        there and overwrite what lay behind (the reference's truncate_kv,
        crates/core/src/backend.rs:129-310, crates/backends/backend_common/src/cpu_backend.rs:527-543,
        crates/backends/backend_common/src/kv_cache.rs:389-397). Pages wholly behind the new
        length go back to the pool. Refused where it cannot be done: beyond the present length,
        into keys that a windowed group has already given up, or with per-sequence state."""
        self.cache.truncate(slot, int(length))

    # ---- the step
    accepts_device_tokens = True
    hands_out_copies = True         # `step(..., keep_logits=False)` gives the rows themselves

    def step(self, entries, tokens_on_device=None, keep_logits=True):
        """Run the entries' tokens; returns float32 logits [wanted, vocab] on the GPU
        (rows in the order of the entries and of their `want`), or None if nothing is wanted.
        A step in which every sequence brings one token and wants its logits writes them into a
        buffer of the engine's that the next such step writes again; what is returned is a copy
        of the caller's own, unless `keep_logits` is false: then it is a view of that buffer, for
        callers that are done with it before their next step (the generation loop).
        `tokens_on_device` (int32 [entries] on the GPU, every entry bringing one token): the
        tokens are taken from there, in the stream's order, and the entries' own are only
        placeholders; so a step can be put on the stream before the host has seen the tokens
        that the step before it chose."""
        if not entries:
            raise RequestError("a step needs at least one sequence")
        if tokens_on_device is not None:
            if (tokens_on_device.dtype != torch.int32 or tuple(tokens_on_device.shape) != (len(entries),)
                    or tokens_on_device.device != self.device or any(len(e.tokens) != 1 for e in entries)):
                raise RequestError("tokens_on_device must be int32 [entries] on the engine's GPU, for entries "
                                   "of one token each")
        vocab = self.spec.vocab_size
        seen = set()
        starts = []
        for e in entries:
            if e.slot in seen:
                raise RequestError(f"slot {e.slot} appears twice in one step")
            seen.add(e.slot)
            if len(e.tokens) == 0:
                raise RequestError("a sequence of a step has no tokens")
            if len(e.tokens) == 1:              # decoding: no array for one number
                low = high = e.tokens[0]
                if not isinstance(low, (int, np.integer)) or isinstance(low, bool):
                    raise RequestError("token ids must be integers")
            else:
                ids = np.asarray(e.tokens)
                if ids.dtype.kind not in "iu":
                    raise RequestError("token ids must be integers")
                low, high = int(ids.min()), int(ids.max())
            if low < 0 or high >= vocab:
                raise RequestError(f"token id {low if low < 0 else high} out of range (vocab_size {vocab})")
            for j in e.want:
                if not 0 <= int(j) < len(e.tokens):
                    raise RequestError(f"wanted place {j} is outside the sequence's "
                                       f"{len(e.tokens)} tokens")
            start = self.cache.length(e.slot)
            if start + len(e.tokens) > self.spec.max_positions:
                raise RequestError(f"sequence of {start + len(e.tokens)} tokens exceeds "
                                   f"max_position_embeddings ({self.spec.max_positions})")
            starts.append(start)
        # all pages of the step or none: a step that does not fit leaves the cache as it was
        self.cache.reserve_all([(e.slot, len(e.tokens)) for e in entries])
        # fixed-size state is changed in place by the parts: what the step's slots hold is set aside
        # first, so that a step that fails leaves them as they were (nothing for a cache without state)
        state_before = self.cache.save_state([e.slot for e in entries])
        try:
            if self.static_decode and all(len(e.tokens) == 1 and list(e.want) == [0] for e in entries):
                logits = self._decode_step(entries, starts, tokens_on_device)
                if keep_logits:
                    logits = logits.clone()
            else:
                meta = batching.pack(entries, starts, self.device)
                if tokens_on_device is not None:
                    meta.token_ids.copy_(tokens_on_device)
                logits = self.model.forward(self.rt, meta, self.cache)
        except Exception:
            for e in entries:       # nothing was committed: give back what was taken for the step
                self.cache.unreserve(e.slot)
            self.cache.restore_state(state_before)
            raise
        for e in entries:
            self.cache.commit(e.slot, len(e.tokens))
        self.steps_run += 1
        return logits

    def _decode_step(self, entries, starts, tokens_on_device=None):
        """One token for each sequence, every logit wanted: the launch-bound case. The step's
        metadata lives in fixed buffers, and the forward pass of a shape is recorded into a HIP graph
        that is replayed from then on, so that the host launches one graph and not hundreds of
        kernels. The step runs at the size of a ladder at or above its sequences
        (batch.decode_batch_bucket), filled up with padding rows in the cache's padding slot: a batch
        whose sequences end one after another then meets few new shapes instead of one a sequence.
        A graph is tied to that batch size, to the bucket of the longest context (which sizes the
        attention grid) and to whether the contexts are of very unequal lengths (the attention then
        deals its grid out by a list). All graphs write their logits into the first rows of the
        engine's one buffer; what is returned here is a view of those rows, which the next decode
        step writes again (`step` copies it for callers that keep it). At most MAX_GRAPHS graphs and
        MAX_DECODE_BATCH_SIZES batch sizes are kept, the least recently used go first."""
        n = len(entries)
        B = decode_batch_bucket(n)          # the step runs at this size, the rows beyond n are padding
        state = self._decode.get(B)
        if state is None:
            if len(self._decode) >= MAX_DECODE_BATCH_SIZES:
                torch.cuda.synchronize(self.device)
                old, _ = self._decode.popitem(last=False)
                for key in [k for k in self._graphs if k[0] == old]:
                    del self._graphs[key]
            held = 0 if self._shared_logits is None else self._shared_logits.shape[0]
            if B > held:
                torch.cuda.synchronize(self.device)     # nothing that writes the old buffer still runs
                self._graphs.clear()
                self._decode.clear()
                rows = max(B, min(decode_batch_bucket(self.cache.n_slots), max(SHARED_LOGITS_ROWS, 2 * held)))
                self._shared_logits = None
                self._shared_logits = torch.empty((rows, self.spec.vocab_size), dtype=torch.float32,
                                                  device=self.device)
            state = self._decode[B] = _DecodeState(StaticDecodeMeta(B, self.device, self.cache.pad_slot),
                                                   self._shared_logits[:B])
        self._decode.move_to_end(B)
        meta = state.static.update(entries, starts)
        if tokens_on_device is not None:
            meta.token_ids[:n].copy_(tokens_on_device)      # behind the copy from the host, before the graph
        if not self.use_graphs:
            return self.model.forward(self.rt, meta, self.cache, logits_out=state.logits)[:n]
        key = (B, meta.context_bucket, meta.unequal)
        graph = self._graphs.get(key)
        if graph is not None:
            self._graphs.move_to_end(key)
            graph.replay()
            return state.logits[:n]
        if B > self._sized_rows:
            # no step this large has run yet: it runs as it is, which also sizes every scratch buffer
            self._sized_rows = B
            return self.model.forward(self.rt, meta, self.cache, logits_out=state.logits)[:n]
        if len(self._graphs) >= MAX_GRAPHS:
            torch.cuda.synchronize(self.device)      # no graph that is dropped here still runs
            while len(self._graphs) >= MAX_GRAPHS:
                self._graphs.popitem(last=False)
        # A shape no larger than one that has run before is recorded at once, without a pass of its
        # own outside a graph: the buffers are there. Where one turns out to be missing after all (a
        # longer context's partial results, a list of ranges), the recording is given up and the
        # step runs as it is; the shape's next step is then recorded.
        # Recorded on a stream of its own behind what the step's stream holds, without waiting for
        # the GPU: the host records the kernels while the steps before still run. (torch.cuda.graph
        # as a context would first wait for the GPU and hand every cached block back to the driver.)
        graph = torch.cuda.CUDAGraph()
        if self._capture_stream is None:
            self._capture_stream = torch.cuda.Stream(self.device)
        step_stream = torch.cuda.current_stream(self.device)
        self._capture_stream.wait_stream(step_stream)
        try:
            with torch.cuda.stream(self._capture_stream):
                graph.capture_begin()
                try:
                    self.model.forward(self.rt, meta, self.cache, logits_out=state.logits)
                finally:
                    graph.capture_end()
        except NeedsEagerStep:
            step_stream.wait_stream(self._capture_stream)
            del graph
            return self.model.forward(self.rt, meta, self.cache, logits_out=state.logits)[:n]
        except Exception:
            # Nothing of a failed recording has run. The two streams are joined again, and the shape
            # starts over: its next step runs as it is (which shows the same failure outside a
            # recording) instead of failing in a recording again at every step.
            step_stream.wait_stream(self._capture_stream)
            self._sized_rows = 0
            raise
        step_stream.wait_stream(self._capture_stream)
        self._graphs[key] = graph
        self.graphs_captured += 1
        graph.replay()
        return state.logits[:n]

    def decode_graph_stats(self):
        """(graphs kept, batch sizes kept, bytes of the decode steps' logits buffers)."""
        held = 0 if self._shared_logits is None else self._shared_logits.numel() * 4
        return len(self._graphs), len(self._decode), held

    def generate(self, prompts, params=None, max_batch=64, on_token=None, interrupt=None, prefill_chunk=None):
        """Generate from lists of token ids; see engine.generate.Generator."""
        from .generate import Generator
        gen = Generator(self, max_batch=max_batch, prefill_chunk=prefill_chunk)
        results = gen.generate(prompts, params, on_token, interrupt)
        self.last_generation_stats = gen.stats
        return results
