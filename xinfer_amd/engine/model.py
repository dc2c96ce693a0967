"""The architecture-neutral model: embedding, blocks in schedule order, final norm, head.

Built from a `ModelSpec` alone.  The reference's counterpart is Qwen3ForCausalLM
(/root/reference/src/models/qwen3.rs:137-445; forward_inner 311-374): embed, the layer
loop, selection of the wanted rows, final norm, lm_head with float32 logits.  Unlike the
reference, which keeps only the last row of each sequence (qwen3.rs:359-363), any set of
rows may be asked for.
"""
from __future__ import annotations

import sys
from dataclasses import dataclass
from typing import Dict, List, Tuple

import torch

from ..config.spec import ModelSpec
from ..parts import (KVNeed, LayerCache, StateNeed, StepContext, Stream, block_class, embedding_class,
                     head_class, norm_class, state_needs_of, stream_op_class)

EMBEDDING_CACHE = -1        # the key of the state that the embedding keeps (no layer's index, no run's cache id)
from ..weights.store import TensorDecl, WeightStore


@dataclass(frozen=True)
class CacheGroupNeed:
    """Layers whose cache needs are the same kind: all keys (window 0) or a window."""
    window: int
    layers: Tuple[int, ...]             # keys of the caches in this group (layer indices, or runs' cache ids)


class CausalLM:
    def __init__(self, spec: ModelSpec, dtype: torch.dtype):
        if dtype not in (torch.float32, torch.bfloat16):
            raise ValueError(f"dtype {dtype} is not supported (float32 or bfloat16)")
        self.spec = spec
        self.dtype = dtype
        self.embedding = embedding_class(spec.embedding.kind)(spec.embedding, dtype)
        self.blocks = [block_class(l.block)(l, dtype) for l in spec.layers]
        self.final_norm = norm_class(spec.final_norm.kind)(spec.final_norm, dtype)
        self.head = head_class(spec.head.kind)(spec.head, dtype)
        # what runs on the stream before a schedule entry's layer: one object a distinct spec
        self.stream_ops = {}
        for e in spec.schedule:
            if e.before is not None and id(e.before) not in self.stream_ops:
                self.stream_ops[id(e.before)] = stream_op_class(e.before.kind)(e.before, dtype)
        self._keep_first = any(op.needs_first for op in self.stream_ops.values())
        for e in spec.schedule:
            if not (0 <= e.layer < len(self.blocks)):
                raise ValueError(f"schedule names layer {e.layer} but the model has {len(self.blocks)}")
            if e.cache_of is not None and e.cache_id is not None:
                raise ValueError("a schedule entry reads another run's cache or keeps one of its own, not both")
        ids = {e.cache_id for e in spec.schedule if e.cache_id is not None}
        for e in spec.schedule:
            if e.cache_of is not None and e.cache_of not in ids and not (0 <= e.cache_of < len(self.blocks)):
                raise ValueError(f"schedule entry reads the cache of unknown layer {e.cache_of}")
        self._plan_cache()

    @property
    def graph_safe(self) -> bool:
        """Every part can be recorded into a HIP graph (see `Part.graph_safe`)."""
        return all(p.graph_safe for p in (self.embedding, self.final_norm, self.head, *self.blocks, *self.stream_ops.values()))

    # ---- weights -------------------------------------------------------------
    @classmethod
    def declare(cls, spec: ModelSpec) -> List[TensorDecl]:
        decls = embedding_class(spec.embedding.kind).declare(spec.embedding)
        for l in spec.layers:
            decls += block_class(l.block).declare(l)
        for e in spec.schedule:
            if e.before is not None:
                decls += stream_op_class(e.before.kind).declare(e.before, "")
        decls += norm_class(spec.final_norm.kind).declare(spec.final_norm, str(spec.final_norm.get("prefix", "")))
        decls += head_class(spec.head.kind).declare(spec.head)
        seen, out = set(), []
        for d in decls:                      # a tied head names the embedding table again
            if d.name not in seen:
                seen.add(d.name)
                out.append(d)
        return out

    def load(self, store: WeightStore, device) -> "CausalLM":
        # tensors of the source that no part asked for are left alone, as the reference leaves them
        self.ignored_tensors = store.check(self.declare(self.spec))
        if self.ignored_tensors:
            shown = ", ".join(self.ignored_tensors[:4]) + (", ..." if len(self.ignored_tensors) > 4 else "")
            print(f"[xinfer_amd] {store.where}: {len(self.ignored_tensors)} tensors the model does not use "
                  f"are ignored ({shown})", file=sys.stderr, flush=True)
        self.device = torch.device(device)
        self.embedding.load(store, "", device)
        for b in self.blocks:
            b.load(store, device)
        for op in self.stream_ops.values():
            op.load(store, "", device)
        self.final_norm.load(store, str(self.spec.final_norm.get("prefix", "")), device)
        self.head.load(store, "", device, shared=self.embedding.table if self.head.tied else None)
        return self

    # ---- cache planning --------------------------------------------------------
    def _plan_cache(self) -> None:
        """Which runs own pages, in which group; which own per-request state.  A cache is known by a key:
        the layer's index, or the `cache_id` of a run that keeps one of its own."""
        self.kv_needs: Dict[int, KVNeed] = {}
        self.state_needs: Dict[int, StateNeed] = {}      # a cache's state, or a tuple of them if its part keeps several
        layer_of: Dict[int, int] = {}
        for e in self.spec.schedule:
            if e.cache_of is None:
                key = e.layer if e.cache_id is None else e.cache_id
                if layer_of.setdefault(key, e.layer) != e.layer:
                    raise ValueError(f"cache {key} is kept by runs of layers {layer_of[key]} and {e.layer}")
        owners = []
        for e in self.spec.schedule:
            owner = self.cache_key(e)
            if owner not in owners:
                owners.append(owner)
                layer_of.setdefault(owner, owner)      # a cache that is only ever read: laid out as that layer's
        windows: List[int] = []
        by_window: Dict[int, List[int]] = {}
        for key in owners:
            l = layer_of[key]
            kv = self.blocks[l].cache_need()
            if kv is not None:
                self.kv_needs[key] = kv
                if kv.window not in by_window:
                    by_window[kv.window] = []
                    windows.append(kv.window)
                by_window[kv.window].append(key)
            st = self.blocks[l].state_need()
            if st is not None:
                self.state_needs[key] = st
        if state_needs_of(self.embedding.state_need()):
            self.state_needs[EMBEDDING_CACHE] = self.embedding.state_need()
        self.cache_groups: List[CacheGroupNeed] = [
            CacheGroupNeed(w, tuple(by_window[w])) for w in windows]
        self.group_of_layer: Dict[int, int] = {
            l: g for g, grp in enumerate(self.cache_groups) for l in grp.layers}

    @staticmethod
    def cache_key(e) -> int:
        """The key of the cache that a schedule entry's run uses."""
        if e.cache_of is not None:
            return e.cache_of
        return e.layer if e.cache_id is None else e.cache_id

    # ---- step ------------------------------------------------------------------
    def forward(self, ids: torch.Tensor, ctx: StepContext, caches: Dict[int, LayerCache],
                want_rows: torch.Tensor) -> torch.Tensor:
        """ids int32 [T]; caches: layer index -> the cache that layer owns; want_rows int32
        [R].  Returns float32 logits [R, vocab]."""
        if EMBEDDING_CACHE in self.state_needs:
            first = self.embedding.forward(ids, ctx, cache=caches[EMBEDDING_CACHE])
        else:
            first = self.embedding.forward(ids, ctx)
        kept_first = first.clone() if self._keep_first else None       # the norms add into `first` in place
        # an embedding kind may also hand on its result rounded to the activation dtype (`rows`)
        stream = Stream(first, None, rows=getattr(self.embedding, "rows", None))
        schedule = self.spec.schedule
        for i, e in enumerate(schedule):
            c = caches.get(self.cache_key(e))
            if c is None:
                c = LayerCache()
            elif e.cache_of is not None:
                c = LayerCache(c.group, c.pools, c.state, write=False, states=c.states)
            if e.before is not None:
                stream = self.stream_ops[id(e.before)].forward(stream, kept_first, ctx)
            blk = self.blocks[e.layer]
            if getattr(blk, "folds", False):
                # the block that runs next may let this one half do its first norm
                nxt = self.blocks[schedule[i + 1].layer] if i + 1 < len(schedule) else None
                next_norm = nxt.first_norm() if getattr(nxt, "folds", False) else None
                if nxt is not None and schedule[i + 1].before is not None:
                    next_norm = None          # something changes the stream in between: the norm sees another sum
                stream = blk.forward(stream, ctx, c, next_norm=next_norm)
            else:
                stream = blk.forward(stream, ctx, c)
        if stream.pending is not None and stream.pending_scale != 1.0:
            h = self.final_norm.forward(stream.resid, stream.pending, self.dtype, rows=want_rows,
                                        add_scale=stream.pending_scale)
        else:
            h = self.final_norm.forward(stream.resid, stream.pending, self.dtype, rows=want_rows)
        return self.head.forward(h)
