"""Architecture-neutral description of a model as data.

An architecture's typed config turns itself into a `ModelSpec`: a list of layers,
each naming the kind of its mixer, feed-forward, norms and block arrangement with
all sizes and constants as parameters, plus the order in which the layers run.
The parts registry builds the runnable objects from these records, so no part
needs to know which model it belongs to, and layers of one model may differ.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping, Optional, Tuple


@dataclass(frozen=True)
class PartSpec:
    """`kind` selects a class in the registry of its category; `params` are its sizes
    and constants.  `params` is a plain mapping so that a new kind needs no change here."""
    kind: str
    params: Mapping[str, Any] = field(default_factory=dict)

    def __getitem__(self, key: str) -> Any:
        return self.params[key]

    def get(self, key: str, default: Any = None) -> Any:
        return self.params.get(key, default)


@dataclass(frozen=True)
class LayerSpec:
    """One decoder layer: which block arrangement, and the parts it is made of.
    Tensor names are data of the layer too: `prefix` is the prefix of all its weights,
    `mixer_name` and `feed_forward_name` what follows it for those two parts, and the keys
    of `norms` what follows it for each norm.  The order of `norms` says which is which:
    the block arrangement takes them in the order in which it runs them (for "prenorm":
    the norm before the mixer, then the norm before the feed-forward)."""
    prefix: str
    block: str
    mixer: PartSpec
    feed_forward: Optional[PartSpec]      # None: the layer has no feed-forward (block arrangements that allow it)
    norms: Mapping[str, PartSpec]
    mixer_name: str = "self_attn"
    feed_forward_name: str = "mlp"
    block_params: Mapping[str, Any] = field(default_factory=dict)    # constants of the arrangement itself

    def norm_items(self, count: int):
        """The first `count` norms as (tensor name under the prefix, spec), in running order."""
        items = list(self.norms.items())
        if len(items) < count:
            raise ValueError(f"layer {self.prefix!r} names {len(items)} norms; its block arrangement "
                             f"{self.block!r} runs {count}")
        return items[:count]


@dataclass(frozen=True)
class ScheduleEntry:
    """One step of the run order.  `layer` indexes `ModelSpec.layers`; a layer may be
    named more than once.  `cache_of` makes this run read (and not write) the cache
    that another layer's run owns; None means the layer's own.  `cache_id` gives this run a
    cache and state of its own under that number, whatever layer's weights it runs with (a
    layer that is run again with the same tensors, as a layer of its own: ids and the indices
    of layers that own a cache share one numbering, so an id is no such layer's index).  `before`: a stream op
    (a `PartSpec` of that registry) that runs on the residual stream right before this run, e.g. what a pass over a
    span of layers adds to the stream when it starts."""
    layer: int
    cache_of: Optional[int] = None
    cache_id: Optional[int] = None
    before: Optional[PartSpec] = None


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    max_positions: int
    embedding: PartSpec
    layers: Tuple[LayerSpec, ...]
    schedule: Tuple[ScheduleEntry, ...]
    final_norm: PartSpec                  # its parameter "prefix" (default "") is the prefix of its tensors' names
    head: PartSpec
    eos_token_ids: Tuple[int, ...] = ()
