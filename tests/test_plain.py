"""The plain implementation pinned by what fixes it beside the reference's text: library
routines it must reduce to, invariants, and the shapes of the reference's own probes.  Each
check is chosen so that a plausible mistake (a wrong sign or pairing, a norm in the wrong
place, a mask off by one) fails it.  No GPU."""
import math

import pytest
import torch

import plain_qwen3 as plain
from configs import TINY


def test_rmsnorm_is_the_library_routine_and_scale_free():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(5, 48, generator=g, dtype=torch.float64)
    w = torch.randn(48, generator=g, dtype=torch.float64)
    lib = torch.nn.functional.rms_norm(x, (48,), w, 1e-6)
    assert torch.allclose(plain.rms_norm(x, w, 1e-6), lib, rtol=1e-12, atol=1e-12)
    assert torch.allclose(plain.rms_norm(7.0 * x, w, 0.0), plain.rms_norm(x, w, 0.0), rtol=1e-12)
    unit = plain.rms_norm(x, torch.ones(48, dtype=torch.float64), 0.0)
    assert torch.allclose(unit.pow(2).mean(-1), torch.ones(5, dtype=torch.float64))


def test_rope_tables_follow_the_reference_arithmetic():
    """inv_freq is 1f32 / f32(theta^(2i/d)) and the angle a float32 product
    (/root/reference/src/models/layers/rotary_emb.rs:50-56)."""
    cos, sin = plain.rope_tables(1e6, 16, 512)
    assert cos.dtype == torch.float32 and cos.shape == (512, 8)
    i = 3
    inv = torch.tensor(1.0, dtype=torch.float32) / torch.tensor(1e6 ** (2 * i / 16), dtype=torch.float64).to(torch.float32)
    ang = torch.tensor(400.0, dtype=torch.float32) * inv
    assert float(cos[400, i]) == float(torch.cos(ang)) and float(sin[400, i]) == float(torch.sin(ang))
    assert torch.equal(cos[0], torch.ones(8)) and torch.equal(sin[0], torch.zeros(8))


def test_rope_invariants_and_sign():
    g = torch.Generator().manual_seed(8)
    d = 16
    cos, sin = plain.rope_tables(10000.0, d, 128)
    q = torch.randn(1, 1, d, generator=g, dtype=torch.float64)
    k = torch.randn(1, 1, d, generator=g, dtype=torch.float64)
    at = lambda x, p: plain.apply_rope(x, torch.tensor([p]), cos.double(), sin.double())
    assert torch.allclose(at(q, 0), q)                                   # position 0 is the identity
    r = at(q, 37)                                                        # pairs (i, i + d/2) keep their norm
    assert torch.allclose(r[..., :8] ** 2 + r[..., 8:] ** 2, q[..., :8] ** 2 + q[..., 8:] ** 2)
    d1 = (at(q, 9) * at(k, 4)).sum()                                     # only the distance counts
    d2 = (at(q, 59) * at(k, 54)).sum()
    assert abs(float(d1 - d2)) < 1e-5
    assert abs(float((at(q, 9) * at(k, 4)).sum() - (at(q, 9) * at(k, 5)).sum())) > 1e-3
    e = torch.zeros(1, 1, d, dtype=torch.float64)                        # sign: e_0 turns towards e_{d/2}
    e[..., 0] = 1.0
    r = at(e, 1)
    assert abs(float(r[0, 0, 0]) - math.cos(1.0)) < 1e-6 and abs(float(r[0, 0, 8]) - math.sin(1.0)) < 1e-6


def test_rope_on_the_reference_probe_shapes():
    """q (11,3,8), k (11,2,8), tables (64,4), the probe's positions
    (/root/reference/tests/probes/attention_misc_precision_probe.rs:36-40); compared with the
    probe's golden formula written out element by element."""
    g = torch.Generator().manual_seed(1)
    pos = torch.tensor([0, 7, 2, 31, 9, 16, 3, 63, 4, 12, 5])
    cos, sin = plain.rope_tables(10000.0, 8, 64)
    assert cos.shape == (64, 4)
    q = torch.randn(11, 3, 8, generator=g)
    out = plain.apply_rope(q, pos, cos, sin)
    for t in (1, 7):
        for h in (0, 2):
            for i in range(4):
                c, s = cos[pos[t], i], sin[pos[t], i]
                assert torch.allclose(out[t, h, i], q[t, h, i] * c - q[t, h, i + 4] * s)
                assert torch.allclose(out[t, h, i + 4], q[t, h, i] * s + q[t, h, i + 4] * c)


def test_attention_is_the_library_routine():
    g = torch.Generator().manual_seed(10)
    T, nq, nkv, d = 12, 6, 2, 8
    q = torch.randn(T, nq, d, generator=g, dtype=torch.float64)
    k = torch.randn(T, nkv, d, generator=g, dtype=torch.float64)
    v = torch.randn(T, nkv, d, generator=g, dtype=torch.float64)
    out = plain.attention(q, k, v)
    lib = torch.nn.functional.scaled_dot_product_attention(
        q.transpose(0, 1)[None], k.transpose(0, 1)[None], v.transpose(0, 1)[None], is_causal=True,
        enable_gqa=True)[0].transpose(0, 1)
    assert torch.allclose(out, lib, rtol=1e-10, atol=1e-12)
    assert torch.allclose(plain.attention(q[:1], k[:1], v[:1])[0, 0], v[0, 0])     # one token gives v
    # head h reads kv head h // group: swapping the kv heads swaps the two halves of the q heads
    sw = plain.attention(torch.cat([q[:, 3:], q[:, :3]], 1), k.flip(1), v.flip(1))
    assert torch.allclose(torch.cat([sw[:, 3:], sw[:, :3]], 1), out)


def test_window_sees_exactly_w_keys():
    g = torch.Generator().manual_seed(11)
    T, d, w, p = 12, 8, 5, 9
    q = torch.randn(T, 1, d, generator=g, dtype=torch.float64)
    k = torch.randn(T, 1, d, generator=g, dtype=torch.float64)
    v = torch.randn(T, 1, d, generator=g, dtype=torch.float64)
    out = plain.attention(q, k, v, window=w)
    s = (q[p, 0] @ k[p - w + 1:p + 1, 0].T) / math.sqrt(d)
    assert torch.allclose(out[p, 0], torch.softmax(s, -1) @ v[p - w + 1:p + 1, 0])
    assert torch.allclose(plain.attention(q, k, v, window=T), plain.attention(q, k, v))


def test_swiglu_is_the_library_routine():
    g = torch.Generator().manual_seed(4)
    a = torch.randn(13, 48, generator=g, dtype=torch.float64)      # the probe's shape (13, 48)
    b = torch.randn(13, 48, generator=g, dtype=torch.float64)
    assert torch.allclose(plain.swiglu(a, b), torch.nn.functional.silu(a) * b, rtol=1e-12, atol=1e-14)
    assert float(plain.swiglu(torch.zeros(1, dtype=torch.float64), torch.ones(1, dtype=torch.float64))) == 0.0


def _tiny_weights(name, tmp_path):
    from xinfer_amd.weights import write_random_model
    t = TINY[name]
    d = write_random_model(str(tmp_path / name), t["config"], t["seed"], t["linear_std"], t["norm_std"])
    return plain.PlainModel(d, torch.float64)


def test_zero_layers_is_norm_and_head(tmp_path):
    pm = _tiny_weights("A", tmp_path)
    c = dict(pm.config, num_hidden_layers=0)
    ids = [3, 200, 17]
    W = pm.weights
    x = W["model.embed_tokens.weight"][torch.tensor(ids)]
    want = plain.rms_norm(x, W["model.norm.weight"], c["rms_norm_eps"]) @ W["model.embed_tokens.weight"].T
    assert torch.allclose(plain.model_logits(c, W, ids).double(), want, atol=1e-6)     # tied head = embedding


def test_causality_and_position_shift(tmp_path):
    """Logits at a position do not depend on later tokens; and because only distances count
    in rotary attention, a sequence placed at another starting position gives the same logits."""
    pm = _tiny_weights("B", tmp_path)
    ids = [5, 77, 300, 41, 9, 500, 123, 8]
    full = pm.logits(ids)
    assert torch.allclose(full[:5], pm.logits(ids[:5]), atol=1e-9)
    shifted = plain.model_logits(pm.config, pm.weights, ids, start=100)
    assert torch.allclose(full, shifted, atol=2e-4)          # angles are float32: equal to rounding
    assert not torch.allclose(full[1:], plain.model_logits(pm.config, pm.weights, ids[1:]), atol=1e-3)


def test_layer_order_norm_before_mixer(tmp_path):
    """A norm in the wrong place fails this: scaling the input embedding of a one-layer model
    leaves the attention branch unchanged (pre-norm), so logits change only through the
    residual path; with eps -> 0 and the final norm, the logits are scale-free altogether."""
    pm = _tiny_weights("A", tmp_path)
    c = dict(pm.config, num_hidden_layers=1, rms_norm_eps=0.0)
    W = dict(pm.weights)
    ids = [1, 2, 3, 4]
    base = plain.model_logits(c, W, ids)
    # make both branch outputs vanish: logits = head(norm(x)) whatever the scale of x
    W2 = dict(W)
    W2["model.layers.0.self_attn.o_proj.weight"] = torch.zeros_like(W["model.layers.0.self_attn.o_proj.weight"])
    W2["model.layers.0.mlp.down_proj.weight"] = torch.zeros_like(W["model.layers.0.mlp.down_proj.weight"])
    a = plain.model_logits(c, W2, ids)
    W2["model.embed_tokens.weight"] = W["model.embed_tokens.weight"]
    x = W["model.embed_tokens.weight"][torch.tensor(ids)]
    want = plain.rms_norm(x, W["model.norm.weight"], 0.0) @ W["model.embed_tokens.weight"].T
    assert torch.allclose(a.double(), want, atol=1e-6)
    assert not torch.allclose(a, base, atol=1e-4)


def test_bias_is_one_more_input_column(tmp_path):
    """A bias on q, k and v is what a constant input of 1 with the bias as its weight column
    gives: the attention block with `attention_bias` equals the block without, run on [x, 1]
    with weights [W, b].  A bias added after the norm or the rotation, or one on o_proj, fails."""
    pm = _tiny_weights("W", tmp_path)
    c, W = pm.config, pm.weights
    assert c["attention_bias"]
    p = "model.layers.1.self_attn"
    T, H = 9, c["hidden_size"]
    g = torch.Generator().manual_seed(4)
    x = torch.randn(T, H, generator=g, dtype=torch.float64)
    W64 = {k: v.double() for k, v in W.items() if k.startswith(p)}
    assert float(W64[f"{p}.k_proj.bias"].abs().max()) > 0
    positions = torch.arange(3, 3 + T)
    cos, sin = plain.rope_tables(c["rope_theta"], c["head_dim"], 64)
    with_bias = plain.attention_block(x, W64, p, c, positions, cos, sin, None)
    W1 = dict(W64)
    for n in ("q", "k", "v"):
        W1[f"{p}.{n}_proj.weight"] = torch.cat([W64[f"{p}.{n}_proj.weight"], W64[f"{p}.{n}_proj.bias"][:, None]], dim=1)
    x1 = torch.cat([x, torch.ones(T, 1, dtype=torch.float64)], dim=1)
    no_bias = plain.attention_block(x1, W1, p, dict(c, attention_bias=False), positions, cos, sin, None)
    assert torch.allclose(with_bias, no_bias, atol=1e-12)
    assert f"{p}.o_proj.bias" not in W
