"""Plain, slow Qwen3 (dense) on the CPU, written from the reference's formulas.

Whole sequences, no cache, one function per part, float32 (or float64) torch tensor
arithmetic only.  It shares no code with xinfer_amd: it parses config.json itself and
reads weights with the `safetensors` package.  The reference was read, not run; every
function cites the lines it follows.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional

import torch


# ---- configuration ----------------------------------------------------------------
def read_config(model_dir: str) -> dict:
    """Keys as in the reference's Config (/root/reference/src/utils/config.rs:277-330):
    head_dim defaults to hidden/heads (attention.rs:446), rope_theta to 10000
    (rotary_emb.rs:49), tie_word_embeddings to false (qwen3.rs:200-209)."""
    with open(os.path.join(model_dir, "config.json")) as f:
        c = json.load(f)
    c.setdefault("head_dim", None)
    if c["head_dim"] is None:
        c["head_dim"] = c["hidden_size"] // c["num_attention_heads"]
    if c.get("rope_theta") is None:
        c["rope_theta"] = 10000.0
    if c.get("tie_word_embeddings") is None:
        c["tie_word_embeddings"] = False
    return c


def read_weights(model_dir: str, dtype=torch.float32) -> Dict[str, torch.Tensor]:
    from safetensors import safe_open
    out = {}
    with safe_open(os.path.join(model_dir, "model.safetensors"), framework="pt") as f:
        for k in f.keys():
            out[k] = f.get_tensor(k).to(dtype)
    return out


def layer_window(c: dict, i: int) -> Optional[int]:
    """`sliding_window` is handed to every layer's attention when present
    (/root/reference/src/models/qwen3.rs:46); `layer_types`, when present, limits it to
    the layers named "sliding_attention"."""
    w = c.get("sliding_window")
    if w is None:
        return None
    lt = c.get("layer_types")
    if lt is None or lt[i] == "sliding_attention":
        return int(w)
    return None


# ---- parts ---------------------------------------------------------------------------
def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """x * rsqrt(mean(x^2) + eps) * w over the last axis, plain weight (no +1).
    /root/reference/src/models/layers/others.rs:22-46 (NormX::forward), eps cast at :275;
    weight without +1 for Qwen3: /root/reference/src/models/layers/attention.rs:491."""
    var = x.pow(2).mean(dim=-1, keepdim=True)
    return x * torch.rsqrt(var + eps) * w


def rope_tables(theta: float, rot: int, max_pos: int):
    """inv_freq[i] = 1f32 / (f32)(theta^(2i/rot)), the power in float64; angle = (f32)p *
    inv_freq in float32; cos and sin of that.
    /root/reference/src/models/layers/rotary_emb.rs:47-61."""
    inv = []
    for i in range(0, rot, 2):
        p = torch.tensor(theta ** (i / rot), dtype=torch.float64).to(torch.float32)
        inv.append(torch.tensor(1.0, dtype=torch.float32) / p)
    inv_freq = torch.stack(inv)                                   # [rot/2] float32
    t = torch.arange(max_pos, dtype=torch.float32)
    freqs = t[:, None] * inv_freq[None, :]                        # float32
    return freqs.cos(), freqs.sin()


def _f32(v) -> torch.Tensor:
    return torch.tensor(v, dtype=torch.float32)


def scaled_rope_tables(c: dict):
    """cos and sin [positions, rot / 2] under config.json's `rope_scaling` (or `rope_parameters`)
    and `partial_rotary_factor`, after ScalingRotaryEmbedding::new,
    /root/reference/src/models/layers/rotary_emb.rs:126-415 and (YaRN) 440-540.  rot =
    int(partial_rotary_factor * head_dim) (:138-141).  The length the model was trained at is
    `original_max_position_embeddings`, else max_position_embeddings / factor, else
    max_position_embeddings (:152-166).  Rows: the positions the model can run, which for YaRN
    over a given original length is round(original * factor) if that is more
    (/root/reference/src/utils/mod.rs:873-897); the reference builds more rows than it can reach."""
    d, theta, max_pos = c["head_dim"], float(c["rope_theta"]), int(c["max_position_embeddings"])
    rot = int(c["partial_rotary_factor"] * d) if c.get("partial_rotary_factor") is not None else d
    rs = c.get("rope_scaling") or c.get("rope_parameters")
    kind = None if rs is None else rs.get("rope_type", rs.get("type"))
    if kind in (None, "default"):
        return rope_tables(theta, rot, max_pos)
    factor = rs.get("factor")
    if rs.get("original_max_position_embeddings") is not None:
        orig = float(rs["original_max_position_embeddings"])
    elif factor is not None:
        orig = max_pos / float(factor)
    else:
        orig = float(max_pos)

    def plain_inv(base: float):          # :116-121
        return [_f32(1.0) / torch.tensor(base ** (i / rot), dtype=torch.float64).to(torch.float32) for i in range(0, rot, 2)]

    rows, mscale = max_pos, None
    if kind == "linear":                 # :172-206: the tensor of frequencies times (f32)(1 / factor)
        inv = [f * _f32(1.0 / float(factor)) for f in plain_inv(theta)]
    elif kind == "llama3":               # :208-282
        lo, hi = float(rs["low_freq_factor"]), float(rs["high_freq_factor"])
        low_wavelen, high_wavelen = _f32(orig / lo), _f32(orig / hi)
        inv = []
        for f in plain_inv(theta):
            wavelen = _f32(2.0) * _f32(math.pi) / f
            if wavelen < high_wavelen:
                inv.append(f)
            elif wavelen > low_wavelen:
                inv.append(f / _f32(float(factor)))
            else:
                smooth = (_f32(orig) / wavelen - _f32(lo)) / _f32(hi - lo)
                inv.append((_f32(1.0) - smooth) * f / _f32(float(factor)) + smooth * f)
    elif kind == "dynamic":              # :284-335
        if rs.get("alpha") is not None:
            base = (theta * float(rs["alpha"])) ** (rot / (rot - 2))
        else:
            fct = float(factor)
            max_len = int(orig * fct)
            base = (theta * ((fct * max_len / orig) - (fct - 1.0))) ** (rot / (rot - 2))
        inv = plain_inv(base)
    elif kind == "yarn":                 # :336-401 and 482-540: everything in float32
        fct = _f32(float(factor))
        beta_fast, beta_slow = float(rs.get("beta_fast", 32.0)), float(rs.get("beta_slow", 1.0))
        extrapolation, attn = float(rs.get("extrapolation_factor", 1.0)), float(rs.get("attn_factor", 1.0))
        base = _f32(theta)
        pw = [torch.pow(base, _f32(float(i)) / _f32(float(rot))) for i in range(0, rot, 2)]
        extra = [_f32(1.0) / p_ for p_ in pw]
        inter = [_f32(1.0) / (fct * p_) for p_ in pw]

        def correction_dim(num_rot: float):      # :441-449
            return (_f32(float(rot)) * torch.log(_f32(orig) / (_f32(num_rot) * _f32(2.0) * _f32(math.pi)))) / (_f32(2.0) * torch.log(base))

        low = max(float(torch.floor(correction_dim(beta_fast))), 0.0)            # :451-463
        high = min(float(torch.ceil(correction_dim(beta_slow))), rot - 1.0)
        if low == high:                                                            # :465-468
            high += 0.001
        inv = []
        for j in range(rot // 2):
            ramp = torch.clamp((_f32(float(j)) - _f32(low)) * _f32(1.0 / (high - low)), 0.0, 1.0)
            mask = (_f32(1.0) - ramp) * _f32(extrapolation)
            inv.append(inter[j] * (_f32(1.0) - mask) + extra[j] * mask)
        mscale = (_f32(1.0) if float(fct) <= 1.0 else _f32(0.1) * torch.log(fct) + _f32(1.0)) * _f32(attn)   # :474-479, 531
        if rs.get("original_max_position_embeddings") is not None and float(factor) > 1.0:
            rows = max(max_pos, int(round(orig * float(factor))))
    else:
        raise ValueError(f"Unknown rope_type: {kind}")
    inv_freq = torch.stack([torch.as_tensor(f, dtype=torch.float32) for f in inv])
    freqs = torch.arange(rows, dtype=torch.float32)[:, None] * inv_freq[None, :]
    cos, sin = freqs.cos(), freqs.sin()
    if mscale is not None:
        cos, sin = cos * mscale, sin * mscale
    return cos, sin


def apply_rope(x: torch.Tensor, positions: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """Non-interleaved ("neox") rotation of the first rot = 2 * cos.shape[1] dims: for i < rot/2,
    o[i] = x[i]*cos - x[i+rot/2]*sin;  o[i+rot/2] = x[i]*sin + x[i+rot/2]*cos; dims from rot on
    pass unchanged.  x: [T, heads, d].  Golden formula of the reference's own probe:
    /root/reference/tests/probes/compare_attention_misc_probe.py:33-49 (else branch);
    Qwen3 uses this layout (is_rope_i = false, /root/reference/src/utils/mod.rs:2303).  The partial
    form is applied by a kernel outside the reference's tree (rotary_emb.rs:87-98): rotating the
    leading dims is the convention of the models that have the factor; parity unpinned."""
    c = cos[positions].to(x.dtype)[:, None, :]
    s = sin[positions].to(x.dtype)[:, None, :]
    h = cos.shape[-1]
    a, b, rest = x[..., :h], x[..., h:2 * h], x[..., 2 * h:]
    return torch.cat([a * c - b * s, a * s + b * c, rest], dim=-1)


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, window: Optional[int] = None,
              scale: Optional[float] = None) -> torch.Tensor:
    """Causal grouped-query attention of one whole sequence.  q [T, nq, d]; k, v [T, nkv, d].
    Query head h reads kv head h // (nq // nkv) (contiguous groups); scores are
    (q . k) / sqrt(d), keys after the query are masked, softmax in the working precision.
    /root/reference/tests/probes/compare_flashinfer_probe.py:51-73 (dense_fp32), scale
    /root/reference/src/models/layers/attention.rs:691.  With a window w the query at p
    sees keys p-w+1 .. p (the kernel that applies it is outside the reference's tree:
    parity unpinned; this is the convention of flash-style kernels, w keys with itself)."""
    T, nq, d = q.shape
    nkv = k.shape[1]
    g = nq // nkv
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    out = torch.empty_like(q)
    pos = torch.arange(T)
    allowed = pos[None, :] <= pos[:, None]
    if window is not None:
        allowed &= pos[None, :] > pos[:, None] - window
    for h in range(nq):
        j = h // g
        s = (q[:, h, :] @ k[:, j, :].T) * scale
        s = s.masked_fill(~allowed, float("-inf"))
        out[:, h, :] = torch.softmax(s, dim=-1) @ v[:, j, :]
    return out


def swiglu(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """silu(gate) * up with silu(z) = z / (1 + e^-z).
    /root/reference/tests/probes/compare_attention_misc_probe.py:81-86;
    /root/reference/src/models/layers/mlp.rs:627-628."""
    return gate / (1.0 + torch.exp(-gate)) * up


def attention_block(x, W, prefix, c, positions, cos, sin, window):
    """q/k/v projections, per-head q_norm and k_norm before RoPE, RoPE on q and k, causal
    GQA, o_proj.  With `attention_bias` q, k and v have a bias each, o_proj has none.
    /root/reference/src/models/layers/attention.rs:805-828 (projections), 388-399 (the three
    biases), 596-608 (o_proj without), 709-748 (per-head norm on [T*heads, d]), 872-879
    (RoPE), 947-958 (attention), 976 (o_proj)."""
    T = x.shape[0]
    nq, nkv, d = c["num_attention_heads"], c["num_key_value_heads"], c["head_dim"]
    eps = c["rms_norm_eps"]
    q = x @ W[f"{prefix}.q_proj.weight"].T
    k = x @ W[f"{prefix}.k_proj.weight"].T
    v = x @ W[f"{prefix}.v_proj.weight"].T
    has = c.get("qkv_bias") if c.get("qkv_bias") is not None else c.get("attention_bias")
    if has is None:                      # neither key: the biases are taken if they are there (attention.rs:472-476, 388-399)
        has = f"{prefix}.q_proj.bias" in W
    if has:
        q = q + W[f"{prefix}.q_proj.bias"]
        k = k + W[f"{prefix}.k_proj.bias"]
        v = v + W[f"{prefix}.v_proj.bias"]
    q, k, v = q.reshape(T, nq, d), k.reshape(T, nkv, d), v.reshape(T, nkv, d)
    q = rms_norm(q, W[f"{prefix}.q_norm.weight"], eps)
    k = rms_norm(k, W[f"{prefix}.k_norm.weight"], eps)
    q = apply_rope(q, positions, cos, sin)
    k = apply_rope(k, positions, cos, sin)
    a = attention(q, k, v, window)
    return a.reshape(T, nq * d) @ W[f"{prefix}.o_proj.weight"].T


def mlp_block(x, W, prefix):
    """down(silu(gate(x)) * up(x)).  /root/reference/src/models/layers/mlp.rs:613-633."""
    g = x @ W[f"{prefix}.gate_proj.weight"].T
    u = x @ W[f"{prefix}.up_proj.weight"].T
    return swiglu(g, u) @ W[f"{prefix}.down_proj.weight"].T


def decoder_layer(x, W, i, c, positions, cos, sin):
    """x -> rms_in -> attn -> (+x) -> rms_post -> mlp -> (+r).
    /root/reference/src/models/qwen3.rs:108-134."""
    p = f"model.layers.{i}"
    eps = c["rms_norm_eps"]
    h = rms_norm(x, W[f"{p}.input_layernorm.weight"], eps)
    a = attention_block(h, W, f"{p}.self_attn", c, positions, cos, sin, layer_window(c, i))
    r = x + a
    h2 = rms_norm(r, W[f"{p}.post_attention_layernorm.weight"], eps)
    return r + mlp_block(h2, W, f"{p}.mlp")


def model_logits(c: dict, W: Dict[str, torch.Tensor], ids: List[int], start: int = 0) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence whose first token sits at position `start`.
    Embedding without scaling, the layers, final norm, lm_head (the embedding table when
    tied).  /root/reference/src/models/qwen3.rs:311-374."""
    dtype = W["model.embed_tokens.weight"].dtype
    d = c["head_dim"]
    cos, sin = scaled_rope_tables(c)
    positions = torch.arange(start, start + len(ids))
    x = W["model.embed_tokens.weight"][torch.tensor(ids)]
    for i in range(c["num_hidden_layers"]):
        x = decoder_layer(x, W, i, c, positions, cos.to(dtype), sin.to(dtype))
    h = rms_norm(x, W["model.norm.weight"], c["rms_norm_eps"])
    head = W["model.embed_tokens.weight"] if c["tie_word_embeddings"] else W["lm_head.weight"]
    return (h @ head.T).to(torch.float32)


class PlainModel:
    def __init__(self, model_dir: str, dtype=torch.float32):
        self.config = read_config(model_dir)
        self.weights = read_weights(model_dir, dtype)

    def logits(self, ids: List[int]) -> torch.Tensor:
        return model_logits(self.config, self.weights, ids)

    def greedy(self, prompt: List[int], n: int) -> List[int]:
        ids = list(prompt)
        out = []
        for _ in range(n):
            t = int(self.logits(ids)[-1].argmax())
            out.append(t)
            ids.append(t)
        return out
