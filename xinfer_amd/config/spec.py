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
    feed_forward: PartSpec
    norms: Mapping[str, PartSpec]
    mixer_name: str = "self_attn"
    feed_forward_name: str = "mlp"

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
    that another layer's run owns; None means the layer's own."""
    layer: int
    cache_of: Optional[int] = None


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
