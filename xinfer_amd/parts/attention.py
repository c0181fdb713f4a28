"""Paged grouped-query attention as a mixer.

h -> packed q/k/v projection (+ bias) -> per-head RMSNorm of q and k -> rotation by position ->
keys/values into the paged cache -> causal attention over the cache (all keys, or the
last `window`) -> output projection.  Reference: Attention::forward_with_kv,
/root/reference/src/models/layers/attention.rs:796-977 (projection 805-828, q/k norm
709-748, RoPE 872-879, paged attention 947-958, o_proj 976); q, k, v weights are
concatenated at load as in attention.rs:376-407.
"""
from __future__ import annotations

from typing import List, Optional

import torch

from .. import kernels
from ..config.spec import PartSpec
from ..weights.store import TensorDecl, WeightStore
from .base import (Folded, KVNeed, LayerCache, Mixer, StepContext, position_encoding_class,
                   register_mixer)
from .linear import Linear


@register_mixer("attention")
class PagedAttention(Mixer):
    VECTOR_MIN_DECODE = 512      # decoded tokens lie in a page each: the form with one wave per head stays ahead up to here
    DECODE_PACKED = True         # steps of single tokens: norm, rotation and cache write inside the attention kernel

    def __init__(self, spec: PartSpec, dtype: torch.dtype):
        super().__init__(spec, dtype)
        self.hidden = int(spec["hidden_size"])
        self.nq = int(spec["num_heads"])
        self.nkv = int(spec["num_kv_heads"])
        self.d = int(spec["head_dim"])
        self.bias = bool(spec.get("bias", False))
        self.qk_norm = bool(spec.get("qk_norm", False))
        self.qk_norm_eps = float(spec.get("qk_norm_eps", 1e-6))
        self.window = int(spec.get("window") or 0)
        self.scale = float(spec.get("scale", self.d ** -0.5))
        if self.nq % self.nkv:
            raise ValueError(f"{self.nq} query heads are not a multiple of {self.nkv} kv heads")
        # A step of single tokens reads nothing on the host where the split-K decode kernel or the
        # generic kernel serves it; sizes that only the prefill kernel takes (more than 16 query heads
        # per kv head) need the step's lengths on the host to lay out its tiles.
        self.graph_safe = dtype != torch.bfloat16 or kernels.decode_attention_takes(self.nq, self.nkv, self.d)
        self.decode_packed = (self.DECODE_PACKED and dtype == torch.bfloat16
                              and kernels.decode_attention_takes(self.nq, self.nkv, self.d))
        pos = spec.get("position")
        self.position = position_encoding_class(pos.kind)(pos, dtype) if pos is not None else None
        self.qkv: Optional[Linear] = None
        self.o: Optional[Linear] = None
        self.q_norm_w = self.k_norm_w = None
        self.qkv_bias = None         # float32 [(nq + 2 nkv) d], added by the kernel after the projection

    # ---- weights -----------------------------------------------------------
    @classmethod
    def declare(cls, spec: PartSpec, prefix: str) -> List[TensorDecl]:
        h, nq, nkv, d = (int(spec[k]) for k in ("hidden_size", "num_heads", "num_kv_heads", "head_dim"))
        out = [TensorDecl(f"{prefix}.q_proj.weight", (nq * d, h)),
               TensorDecl(f"{prefix}.k_proj.weight", (nkv * d, h)),
               TensorDecl(f"{prefix}.v_proj.weight", (nkv * d, h)),
               TensorDecl(f"{prefix}.o_proj.weight", (h, nq * d))]
        if spec.get("bias", False):    # q, k and v only: the reference's o_proj has none (attention.rs:596-608)
            out += [TensorDecl(f"{prefix}.q_proj.bias", (nq * d,)), TensorDecl(f"{prefix}.k_proj.bias", (nkv * d,)),
                    TensorDecl(f"{prefix}.v_proj.bias", (nkv * d,))]
        if spec.get("qk_norm", False):
            out += [TensorDecl(f"{prefix}.q_norm.weight", (d,), "norm"),
                    TensorDecl(f"{prefix}.k_norm.weight", (d,), "norm")]
        return out

    def load(self, store: WeightStore, prefix: str, device) -> None:
        def lin(name):
            t = store.get(name, None, device)
            return t.to(self.dtype) if (self.dtype == torch.float32 or t.dtype != torch.float32) else t
        parts = [lin(f"{prefix}.{n}_proj.weight") for n in ("q", "k", "v")]
        common = torch.float32 if any(p.dtype == torch.float32 for p in parts) else parts[0].dtype
        self.qkv = Linear(torch.cat([p.to(common) for p in parts], dim=0))
        self.o = Linear(lin(f"{prefix}.o_proj.weight"))
        if self.bias:
            self.qkv_bias = torch.cat([store.get(f"{prefix}.{n}_proj.bias", torch.float32, device)
                                       for n in ("q", "k", "v")]).contiguous()
        if self.qk_norm:
            self.q_norm_w = store.get(f"{prefix}.q_norm.weight", torch.float32, device).contiguous()
            self.k_norm_w = store.get(f"{prefix}.k_norm.weight", torch.float32, device).contiguous()
        if self.position is not None:
            self.position.load(store, prefix, device)

    # ---- cache ---------------------------------------------------------------
    def cache_need(self) -> KVNeed:
        # the matrix-core kernels of the bfloat16 path read V in groups of eight keys
        return KVNeed.keys_values(self.nkv, self.d, self.window, v_grouped=self.dtype == torch.bfloat16)

    # ---- step ----------------------------------------------------------------
    takes_sink = True
    takes_folded = True

    def forward(self, x, ctx: StepContext, cache: LayerCache, sink=None):
        """`x`: rows or a `Folded`; `sink`: see `Part.takes_sink`."""
        # a decode step of 17 to 256 rows: the tiled split-K product is ahead of the library, and the
        # kernel below adds its partial sums (which the form for prompt portions does not take)
        rows = None if isinstance(x, Folded) else x.shape[0]
        parts = (rows is not None and self.dtype == torch.bfloat16 and ctx.max_q_len == 1
                 and kernels.MID_FROM <= rows <= min(kernels.MID_ROWS, self.VECTOR_MIN_DECODE - 1))
        qkv = self.qkv(x, out_dtype=self.dtype, allow_split=parts)
        pos = self.position
        slots = ctx.slots[cache.group] if cache.write else ctx.no_slots
        vt = self.dtype == torch.bfloat16
        if (vt and ctx.max_q_len == 1 and self.decode_packed
                and kernels.mfma_attention_supported(self.nq, self.nkv, self.d, cache.k.shape[2])):
            # a step of single tokens: the attention kernel norms and rotates its own heads and
            # stores the new keys and values, one launch less in every layer
            a = kernels.attention_decode_packed_bf16(
                qkv, self.q_norm_w, self.k_norm_w, self.qk_norm_eps,
                pos.cos if pos is not None else ctx.empty_f32,
                pos.sin if pos is not None else ctx.empty_f32,
                pos.rotary_dim if pos is not None else 0,
                pos.interleaved if pos is not None else False,
                ctx.positions, slots, cache.k, cache.v, ctx.block_tables[cache.group], ctx.ctx_lens, ctx.max_ctx_len,
                self.nq, self.scale, self.window, bias=self.qkv_bias,
                similar=getattr(ctx, "similar_lengths", False))
            return self.o(a, out_dtype=self.dtype, allow_split=True, sink=sink)
        q = kernels.qk_norm_rope_kv(
            qkv, self.q_norm_w, self.k_norm_w, self.qk_norm_eps,
            pos.cos if pos is not None else ctx.empty_f32,
            pos.sin if pos is not None else ctx.empty_f32,
            pos.rotary_dim if pos is not None else 0,
            pos.interleaved if pos is not None else False,
            ctx.positions, slots, cache.k, cache.v, self.nq, self.nkv, self.d, v_grouped=vt,
            vector_min_tokens=128 if ctx.max_q_len > 1 else self.VECTOR_MIN_DECODE, bias=self.qkv_bias)
        a = kernels.attention(q, cache.k, cache.v, ctx, cache.group, self.scale, self.window, v_grouped=vt)
        return self.o(a, out_dtype=self.dtype, allow_split=True, sink=sink)     # the next norm adds the parts
