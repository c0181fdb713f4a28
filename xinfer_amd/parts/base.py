"""Interfaces of the parts a layer is made of, and the registries that build them.

A part is built from a `PartSpec` (its sizes and constants) and the activation dtype; it
declares the tensors it needs under a name prefix, loads them from a weight store, and
runs on the tokens of one step.  A part never learns which model it is in.

  Mixer            forward(x, ctx, cache) -> y        x, y: [T, hidden]; y may also be a stack
                                                      [P, T, hidden] of float32 partial sums,
                                                      which the next norm adds in order
                   cache_need() -> KVNeed | None      paged keys/values it wants
                   state_need() -> StateNeed | None   fixed-size per-request state it wants
  FeedForward      forward(x, ctx) -> y               (y as for the mixer)
  Norm             forward(resid, add, out_dtype, rows=None, out=None) -> normed
                   resid is the float32 residual stream; `add` (if given) is summed into
                   it first; with `rows` only those rows are produced and resid is not
                   changed.
  PositionEncoding data for the mixer's fused kernel (for "rope": cos/sin tables)
  Block            forward(stream, ctx, cache) -> stream, the arrangement of the above
                   around the residual stream.
  TokenEmbedding   forward(ids, ctx) -> float32 [T, hidden], the start of the residual stream
                   (`ctx` for kinds that need positions or the request; the built-in one
                   ignores it); `table` is what a tied head shares
  Head             forward(h) -> float32 logits [R, vocab]; load(..., shared=) takes the
                   embedding's table when the spec says `tied`

New kinds register themselves with the decorators below; a `PartSpec.kind` then selects
them.  Nothing else in the engine has to change.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, Dict, List, Optional, Sequence, Tuple

import torch

from ..config.spec import LayerSpec, PartSpec
from ..weights.store import TensorDecl, WeightStore


# ---- what a layer may ask of the cache ------------------------------------------------
PAGE = -1      # in a pool's shape: the axis that is as long as a page has tokens
PAGE_BY_8 = -8 # the axis that is an eighth of that (-n: the page's tokens divided by n, which must divide them)


@dataclass(frozen=True)
class PoolNeed:
    """One paged pool of a layer: the runner allocates [pages, *shape] with PAGE replaced by the
    page size (PAGE_BY_8: by an eighth of it), in `dtype` (None: the activation dtype), and hands it to
    the mixer under `name`.  A shape has one such axis."""
    name: str
    shape: Tuple[int, ...]
    dtype: Optional[torch.dtype] = None

    def bytes_per_token(self, element_size: int) -> int:
        n, by = 1, 1
        for s in self.shape:
            if s < 0:
                by = -int(s)
            else:
                n *= int(s)
        return n // by * (element_size if self.dtype is None else torch.tensor([], dtype=self.dtype).element_size())


@dataclass(frozen=True)
class KVNeed:
    """What a mixer keeps in pages: `window` = 0 keeps every token's entry, w > 0 the last w (pages
    that the window has passed go back to the pool while the request runs); `pools` names the
    pools and the shape of a page in each.  `KVNeed.keys_values` is the pair that attention keeps;
    a mixer of another kind may keep one pool (a latent), or pools of different widths."""
    window: int = 0
    pools: Tuple[PoolNeed, ...] = ()

    @staticmethod
    def keys_values(num_kv_heads: int, head_dim: int, window: int = 0, v_grouped: bool = False) -> "KVNeed":
        """K pool "k" [pages, kv_heads, page_size, head_dim]; V pool "v" the same, or with
        `v_grouped` [pages, kv_heads, page_size / 8, head_dim, 8] (eight keys side by side for every dim)."""
        k = PoolNeed("k", (num_kv_heads, PAGE, head_dim))
        v = PoolNeed("v", (num_kv_heads, PAGE_BY_8, head_dim, 8) if v_grouped else (num_kv_heads, PAGE, head_dim))
        return KVNeed(window, (k, v))


@dataclass(frozen=True)
class StateNeed:
    """Fixed-size state per live request: one slot of this shape and dtype."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass
class LayerCache:
    """What one run of a layer gets from the cache.  `write` is False when the run reads
    the cache that another layer's run owns."""
    group: int = -1
    pools: Dict[str, torch.Tensor] = field(default_factory=dict)   # by PoolNeed.name: [pages, *shape]
    state: Optional[torch.Tensor] = None      # [max_requests, *StateNeed.shape]
    write: bool = True

    @property
    def k(self) -> Optional[torch.Tensor]:
        return self.pools.get("k")

    @property
    def v(self) -> Optional[torch.Tensor]:
        return self.pools.get("v")


@dataclass
class StepContext:
    """Everything about one step's batch that parts may read.  Device tensors unless
    marked host."""
    num_tokens: int
    num_seqs: int
    dtype: torch.dtype                         # activation dtype
    device: torch.device
    positions: torch.Tensor                    # int32 [T]   absolute position of each token
    tok_seq: torch.Tensor                      # int32 [T]   row of the batch each token is in
    cu_q: torch.Tensor                         # int32 [B+1] token offsets of the sequences
    ctx_lens: torch.Tensor                     # int32 [B]   cached length after this step
    state_slots: torch.Tensor                  # int64 [B]   per-request state slot
    slots: List[torch.Tensor]                  # per group int64 [T] cache slot of each token
    block_tables: List[torch.Tensor]           # per group int32 [B, max_pages]
    cu_q_host: Sequence[int] = ()              # host copies for choosing kernels
    ctx_lens_host: Sequence[int] = ()
    max_q_len: int = 0
    max_ctx_len: int = 0
    similar_lengths: bool = False              # host: the mean cached length is at least 0.9 of the longest
    no_slots: Optional[torch.Tensor] = None    # int64 [T] of -1: "store nothing"
    empty_f32: Optional[torch.Tensor] = None   # float32 [1, 0]: tables of "no rotation"
    scratch: Dict[Any, Any] = field(default_factory=dict)   # per-step data that kernels derive once


@dataclass
class NormSink:
    """Given to the part that runs before a norm: "add your result into `resid` yourself and
    prepare `norm`'s input".  A part that can (its last product, for few rows) answers with a
    `Folded`; it may always answer with its plain result instead."""
    resid: torch.Tensor                        # float32 [T, H], the residual stream
    norm: "Norm"


@dataclass
class Folded:
    """Rows whose norm is half done by the product before it: the stream already holds the sum,
    `xg` = round(stream * norm.weight) [T, H], `ss` [T, parts] float32 the parts of each row's
    sum of squares.  The product after the norm takes it in place of normed rows and scales its
    own rows by rsqrt(sum(ss) / H + eps) (`kernels.linear_fold_in`)."""
    xg: torch.Tensor
    ss: torch.Tensor
    norm: "Norm"

    def rows(self, dtype: torch.dtype) -> torch.Tensor:
        """The normed rows themselves, for a consumer without the folded product."""
        inv = torch.rsqrt(self.ss.sum(dim=1) / self.xg.shape[1] + self.norm.eps)
        return (self.xg.float() * inv[:, None]).to(dtype)


@dataclass
class Stream:
    """The residual stream between blocks: `resid` float32 [T, H], and a branch output
    `pending` that has not been added to it yet (the next norm adds it in the same
    kernel that norms), or `folded`: the branch output is already added and the next
    norm (`folded.norm`) half done."""
    resid: torch.Tensor
    pending: Optional[torch.Tensor] = None
    folded: Optional[Folded] = None


class Part:
    # True if `forward` reads nothing of the step on the host (no lengths, no device-to-host
    # copies) and launches the same kernels for every step of the same batch size, so that a
    # decode step can be recorded once as a HIP graph and replayed.  Parts that do not say so
    # keep the whole model on the launch-by-launch path.
    graph_safe = False
    # Folding a norm into the products around it (see `Folded`): a mixer or feed-forward whose
    # `forward` takes a keyword `sink: Optional[NormSink]` says `takes_sink`; one whose `forward`
    # takes a `Folded` in place of its input rows says `takes_folded`; a norm that can be folded
    # (a weight vector `weight` in float32, `eps`, `dim`) says `foldable`.
    takes_sink = False
    takes_folded = False
    foldable = False

    def __init__(self, spec: PartSpec, dtype: torch.dtype):
        self.spec = spec
        self.dtype = dtype

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str) -> List[TensorDecl]:
        return []

    def load(self, store: WeightStore, prefix: str, device) -> None:
        pass


class Mixer(Part):
    def cache_need(self) -> Optional[KVNeed]:
        return None

    def state_need(self) -> Optional[StateNeed]:
        return None

    def forward(self, x: torch.Tensor, ctx: StepContext, cache: LayerCache) -> torch.Tensor:
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, x: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        raise NotImplementedError


class Norm(Part):
    def forward(self, resid: torch.Tensor, add: Optional[torch.Tensor], out_dtype: torch.dtype,
                rows: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        raise NotImplementedError


class PositionEncoding(Part):
    """What a mixer reads of it is between the two.  The built-in attention mixer reads a
    rotation: `cos` and `sin`, float32 tables [max_positions, rotary_dim / 2] on the device
    (made in `load`), `rotary_dim` (even, at most the head size) and `interleaved` (pairs
    (2i, 2i+1) instead of (i, i + rotary_dim / 2)); its kernels apply them to q and k."""


class TokenEmbedding(Part):
    table: Optional[torch.Tensor] = None

    def forward(self, ids: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        raise NotImplementedError


class Head(Part):
    tied = False

    def load(self, store: WeightStore, prefix: str, device, shared: Optional[torch.Tensor] = None) -> None:
        raise NotImplementedError

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


class Block:
    """Arrangement of a layer's parts around the residual stream."""

    graph_safe = False

    def __init__(self, layer: LayerSpec, dtype: torch.dtype):
        self.layer = layer
        self.dtype = dtype

    @classmethod
    def declare(cls, layer: LayerSpec) -> List[TensorDecl]:
        raise NotImplementedError

    def load(self, store: WeightStore, device) -> None:
        raise NotImplementedError

    def cache_need(self) -> Optional[KVNeed]:
        return None

    def state_need(self) -> Optional[StateNeed]:
        return None

    def forward(self, stream: Stream, ctx: StepContext, cache: LayerCache) -> Stream:
        raise NotImplementedError


# ---- registries -------------------------------------------------------------------------
MIXERS: Dict[str, type] = {}
FEED_FORWARDS: Dict[str, type] = {}
NORMS: Dict[str, type] = {}
POSITION_ENCODINGS: Dict[str, type] = {}
BLOCKS: Dict[str, type] = {}
EMBEDDINGS: Dict[str, type] = {}
HEADS: Dict[str, type] = {}


def _register(table: Dict[str, type], what: str) -> Callable[[str], Callable[[type], type]]:
    def named(kind: str) -> Callable[[type], type]:
        def deco(cls: type) -> type:
            table[kind] = cls
            cls.kind = kind
            return cls
        return deco
    return named


register_mixer = _register(MIXERS, "mixer")
register_feed_forward = _register(FEED_FORWARDS, "feed-forward")
register_norm = _register(NORMS, "norm")
register_position_encoding = _register(POSITION_ENCODINGS, "position encoding")
register_block = _register(BLOCKS, "block")
register_embedding = _register(EMBEDDINGS, "embedding")
register_head = _register(HEADS, "head")


def _lookup(table: Dict[str, type], what: str, kind: str) -> type:
    try:
        return table[kind]
    except KeyError:
        raise KeyError(f"unknown {what} kind {kind!r} (registered: {', '.join(sorted(table))})") from None


def mixer_class(kind: str) -> type:
    return _lookup(MIXERS, "mixer", kind)


def feed_forward_class(kind: str) -> type:
    return _lookup(FEED_FORWARDS, "feed-forward", kind)


def norm_class(kind: str) -> type:
    return _lookup(NORMS, "norm", kind)


def position_encoding_class(kind: str) -> type:
    return _lookup(POSITION_ENCODINGS, "position encoding", kind)


def block_class(kind: str) -> type:
    return _lookup(BLOCKS, "block", kind)


def embedding_class(kind: str) -> type:
    return _lookup(EMBEDDINGS, "embedding", kind)


def head_class(kind: str) -> type:
    return _lookup(HEADS, "head", kind)
