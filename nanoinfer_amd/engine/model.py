"""A model put together from parts according to a :class:`ModelSpec`, and one forward pass of it
over the tokens of a step.

Order of a pass (src/model/llama.cpp:297-386): embedding, the blocks in the order the spec lists
them, then, on the wanted rows only, the last norm and the output head.  The reference computes
logits for every row and throws most away (src/engine/engine.cpp:310-338).
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..config.spec import ModelSpec
from ..parts.base import CacheNeed, LayerCache, Runtime, flag_of, pending_for
from ..parts.standard import build_part
from ..registry import get_part


class Model:
    def __init__(self, spec: ModelSpec, tensors: Dict[str, torch.Tensor], rt: Runtime):
        self.spec = spec
        self.rt = rt
        self.embedding = build_part("embedding", spec.embedding, tensors, rt)
        self.blocks = [get_part("block", b.kind)(b, tensors, rt) for b in spec.blocks]
        self.final_norm = build_part("norm", spec.final_norm, tensors, rt)
        self.pass_input = None if spec.pass_input is None else build_part("pass_input", spec.pass_input, tensors, rt)
        # a mix of all earlier states of the stream that takes an entry's result's place (None: none)
        self.stream_mix = None if spec.stream_mix is None else build_part("stream_mix", spec.stream_mix, tensors, rt)
        # a function (index of the entry of the order, h) called after every entry with the complete residual
        # stream, for whoever wants to look at a pass layer by layer; None costs nothing
        self.tap = None
        self.head = build_part("head", spec.head, tensors, rt)
        for run in spec.order:
            if not 0 <= run.block < len(self.blocks):
                raise ValueError(f"the order names block {run.block}, the model has {len(self.blocks)}")
            if run.enter is not None and self.pass_input is None:
                raise ValueError(f"an entry of the order adds row {run.enter} of a pass input, the model has none")
        self._needs: Dict[int, CacheNeed] = {}
        # an embedding that keeps something per request (the token before a portion's first) gets a cache of its
        # own behind the layers' and is handed it with every step
        self._embedding_cache = None
        need = getattr(self.embedding, "cache_need", None)
        if need is not None and need() is not None:
            self._embedding_cache = spec.num_caches()
            self._needs[self._embedding_cache] = need()
        writers = set()
        for run in spec.order:
            need = self.blocks[run.block].cache_need()
            if run.cache in self._needs and self._needs[run.cache] != need:
                raise ValueError(f"cache {run.cache} is used by blocks with different needs: "
                                 f"{self._needs[run.cache]} and {need}")
            self._needs[run.cache] = need
            if run.writes_cache:
                writers.add(run.cache)
            elif run.cache not in writers:
                raise ValueError(f"block {run.block} reads cache {run.cache} before any block has written it")
        self.max_positions = spec.max_positions

    def _all_parts(self):
        return [self.embedding, self.final_norm, self.head] + list(self.blocks) + \
            ([] if self.pass_input is None else [self.pass_input]) + ([] if self.stream_mix is None else [self.stream_mix])

    def graph_safe(self) -> bool:
        """Whether a step of this model may be recorded into a HIP graph: every part says of itself
        that its launches depend on device data only (``graph_safe``), never on the host lists."""
        return all(flag_of(p, "graph_safe", False) for p in self._all_parts())

    def eager_portion_from(self) -> Optional[int]:
        """The fewest tokens of a portion from which on some part wants the step run the ordinary way (it reads the
        step's host lists then); None: no part does."""
        asked = [n for n in (getattr(p, "eager_portion_from", None) for p in self._all_parts()) if n is not None]
        return min(asked) if asked else None

    def idempotent(self) -> bool:
        """Whether running the same step twice leaves the caches as running it once does: true of keys
        and values written to their places, not of a per-request state that a part updates in place."""
        return all(flag_of(p, "idempotent", True) for p in self._all_parts())

    def _settled(self, h, pending):
        """A copy of the stream with what is pending added (for :attr:`tap`; the pass itself goes on as it was)."""
        pending = pending_for(None, pending, self.rt.dtype)
        return h.clone() if pending is None else h + pending.to(h.dtype)

    def cache_needs(self) -> Dict[int, CacheNeed]:
        return dict(self._needs)

    def forward(self, ctx, layer_cache, logits_out: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
        """Run the step described by ``ctx``; ``layer_cache(cache_id, writes)`` gives the
        :class:`LayerCache` of an entry of the order.  Returns float32 logits of ``ctx.logit_rows``
        (None when no row is wanted; the caches are filled all the same).  ``logits_out``: float32
        [at least as many rows, vocab] whose first rows are to take the logits, for a head that
        ``writes_into`` a given tensor (any other head returns a tensor of its own)."""
        if self._embedding_cache is not None:
            h = self.embedding.forward(ctx.token_ids, ctx, cache=layer_cache(self._embedding_cache, True))
        else:
            h = self.embedding.forward(ctx.token_ids, ctx)
        # a pass input that adds the embedding's output again is given a copy of it (the stream itself moves on)
        embedded = h.clone() if getattr(self.pass_input, "wants_embedding", False) else None
        pending = None
        order = self.spec.order
        T = h.shape[0]
        history = None
        if self.stream_mix is not None:
            # every state of the stream is kept for the step: row 0 the embedding's output, row i + 1 the result of
            # entry i, which works in place on the row that was filled with what it reads
            history = torch.empty(len(order) + 1, T, h.shape[1], dtype=torch.float32, device=h.device)
            history[0].copy_(h)
            if order:
                history[1].copy_(h)
                h = history[1]
        for i, run in enumerate(order):
            cache: LayerCache = layer_cache(run.cache, run.writes_cache)
            block = self.blocks[run.block]
            if run.enter is not None:
                if pending is not None:        # the stream has to be complete before a row is added to it
                    h = self.pass_input.settle(h, pending_for(None, pending, self.rt.dtype))
                    pending = None
                h = self.pass_input.forward(h, run.enter) if embedded is None else self.pass_input.forward(h, run.enter, embedded)
            # what the block behind this one would like to find beside the stream (its first norm's input half
            # done by this block's last product), if both blocks know of that
            wants = getattr(self.blocks[order[i + 1].block], "wants_scaled", None) if i + 1 < len(order) and history is None else None
            leave = wants(T) if wants is not None and getattr(block, "leaves_for_next", False) else None
            if leave is not None:
                h, pending = block.forward(h, pending, ctx, cache, leave=leave)
            else:
                h, pending = block.forward(h, pending, ctx, cache)
            if history is not None:
                if pending is not None:        # the entry's result has to be complete before it is mixed
                    h = self.stream_mix.settle(h, pending_for(None, pending, self.rt.dtype))
                    pending = None
                if h.data_ptr() != history[i + 1].data_ptr():     # a block that did not work in place
                    history[i + 1].copy_(h)
                h = self.stream_mix.forward(history, i, out=history[i + 2] if i + 1 < len(order) else None)
            if self.tap is not None:
                self.tap(i, h if pending is None else self._settled(h, pending))
        if ctx.logit_rows is None or ctx.logit_rows.shape[0] == 0:
            return None
        x = self.final_norm.forward(h, pending_for(self.final_norm, pending, self.rt.dtype), rows=ctx.logit_rows)
        if logits_out is not None and getattr(self.head, "writes_into", False):
            return self.head.forward(x, out=logits_out[:x.shape[0]])
        return self.head.forward(x)
