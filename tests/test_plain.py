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


def _scaled(scaling=None, **kw):
    c = dict(head_dim=128, rope_theta=1e6, max_position_embeddings=4096)
    c.update(kw)
    if scaling is not None:
        c["rope_scaling"] = scaling
    return plain.scaled_rope_tables(c)


def test_rope_scaling_linear_and_dynamic_reduce_to_plain_tables():
    """Linear scaling by a power of two puts the plain table's row p at row factor * p, exactly
    (a product with the factor instead of its inverse fails); dynamic scaling is the plain table of
    a larger base, (theta * alpha)^(rot / (rot - 2)) or, from a factor, the value of the NTK rule at
    the scaled length (/root/reference/src/models/layers/rotary_emb.rs:172-206, 284-335)."""
    cos0, sin0 = plain.rope_tables(1e6, 128, 4096)
    cos, sin = _scaled(dict(rope_type="linear", factor=4.0))
    assert cos.shape == cos0.shape
    assert torch.equal(cos[0:4096:4], cos0[:1024]) and torch.equal(sin[0:4096:4], sin0[:1024])
    assert not torch.equal(cos[:1024], cos0[:1024])
    cos, sin = _scaled(dict(type="dynamic", alpha=3.0))
    want = plain.rope_tables((1e6 * 3.0) ** (128 / 126), 128, 4096)
    assert torch.equal(cos, want[0]) and torch.equal(sin, want[1])
    # from a factor: the original length is max / factor = 1024, the scaled one 4096
    cos, sin = _scaled(dict(rope_type="dynamic", factor=4.0))
    want = plain.rope_tables((1e6 * (4.0 * 4096 / 1024 - 3.0)) ** (128 / 126), 128, 4096)
    assert torch.equal(cos, want[0]) and torch.equal(sin, want[1])
    assert torch.equal(_scaled(dict(rope_type="default"))[0], cos0) and torch.equal(_scaled(None)[0], cos0)
    with pytest.raises(ValueError, match="Unknown rope_type"):
        _scaled(dict(rope_type="su", factor=2.0))


def test_rope_scaling_llama3_bands():
    """With the published parameters of that rule (factor 8, low 1, high 4 over 8,192 positions,
    base 500,000) wavelengths under 2,048 positions keep their frequency, those over 8,192 have an
    eighth of it, and the ratio falls from one to the other in between: a blend the wrong way
    round jumps at both edges (/root/reference/src/models/layers/rotary_emb.rs:208-282)."""
    c = dict(head_dim=128, rope_theta=500000.0, max_position_embeddings=16384,
             rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                               original_max_position_embeddings=8192))
    cos, sin = plain.scaled_rope_tables(c)
    cos0, sin0 = plain.rope_tables(500000.0, 128, 16384)
    ang, ang0 = torch.atan2(sin[1], cos[1]).double(), torch.atan2(sin0[1], cos0[1]).double()     # row 1 holds the frequencies
    ratio = ang / ang0
    wavelen = 2 * math.pi / ang0
    assert torch.all(ratio[wavelen < 2048] == 1.0) and int((wavelen < 2048).sum()) > 10
    assert torch.allclose(ratio[wavelen > 8192], torch.tensor(0.125, dtype=torch.float64), rtol=1e-5) and int((wavelen > 8192).sum()) > 10
    mid = (wavelen >= 2048) & (wavelen <= 8192)
    assert int(mid.sum()) >= 3
    r = ratio[mid]
    assert torch.all(r[1:] < r[:-1]) and float(r[0]) < 1.0 and float(r[-1]) > 0.125
    # continuous at the edges: the first blended ratio is near 1, the last near 1/8
    smooth = (8192 / wavelen[mid] - 1.0) / 3.0
    assert torch.allclose(r, (1 - smooth) / 8 + smooth, rtol=1e-4)


def test_rope_scaling_yarn_bands_and_magnitude():
    """Qwen3's own long-context setting (base 1e6, head size 128, factor 4 over 32,768 positions):
    the blend runs over frequencies 23 to 40 (floor and ceil of 128 ln(32768 / (2 pi b)) / (2 ln 1e6)
    for b = 32 and 1).  Below it a frequency stays as it is, above it is a quarter, at 31 it is
    9/17 + (8/17)/4 of itself; cos and sin are scaled by 0.1 ln 4 + 1, times attn_factor.  A ramp the
    wrong way round, a missing magnitude or an original length taken for the scaled one fails
    (/root/reference/src/models/layers/rotary_emb.rs:336-401, 440-540)."""
    rs = dict(rope_type="yarn", factor=4.0, original_max_position_embeddings=32768)
    c = dict(head_dim=128, rope_theta=1e6, max_position_embeddings=40960, rope_scaling=rs)
    cos, sin = plain.scaled_rope_tables(c)
    assert cos.shape == (131072, 64)              # round(32768 * 4) positions, more than max_position_embeddings
    m = 0.1 * math.log(4.0) + 1.0
    assert torch.allclose(cos[:4096] ** 2 + sin[:4096] ** 2, torch.full((4096, 64), m * m), rtol=1e-5)
    cos0, sin0 = plain.rope_tables(1e6, 128, 8)
    freq = torch.atan2(sin[1], cos[1]).double()                      # the angle of position 1
    freq0 = torch.atan2(sin0[1], cos0[1]).double()
    ratio = freq / freq0
    assert torch.allclose(ratio[:24], torch.ones(24, dtype=torch.float64), rtol=1e-5)
    assert torch.allclose(ratio[40:], torch.full((24,), 0.25, dtype=torch.float64), rtol=1e-5)
    assert abs(float(ratio[31]) - (9 / 17 + (8 / 17) / 4)) < 1e-5
    assert torch.all(ratio[24:40][1:] < ratio[24:40][:-1])
    # attn_factor multiplies the magnitude; a factor of 1 is plain RoPE (to the float32 power's rounding)
    cos_a, _ = plain.scaled_rope_tables(dict(c, rope_scaling=dict(rs, attn_factor=1.5)))
    assert torch.allclose(cos_a[:64], cos[:64] * 1.5, rtol=1e-6)
    one = plain.scaled_rope_tables(dict(c, rope_scaling=dict(rope_type="yarn", factor=1.0)))
    ref = plain.rope_tables(1e6, 128, 40960)
    assert one[0].shape == ref[0].shape and torch.allclose(one[0][:512], ref[0][:512], atol=2e-4)
    # without an original length it is max / factor, and the table keeps max_position_embeddings rows
    short = plain.scaled_rope_tables(dict(c, max_position_embeddings=131072, rope_scaling=dict(rope_type="yarn", factor=4.0)))
    assert short[0].shape == (131072, 64) and torch.equal(short[0][:1000], cos[:1000])


def test_partial_rotary_leaves_the_rest_of_a_head_alone(tmp_path):
    """partial_rotary_factor 0.5 of a head of 32: 8 frequencies, dims 16.. pass unchanged and
    dims (i, i + 8) turn together; and a whole model under YaRN and partial rotation still gives
    the same logits wherever the sequence starts (only distances count, also with the scaled
    magnitude)."""
    cos, sin = plain.scaled_rope_tables(dict(head_dim=32, rope_theta=1e4, max_position_embeddings=64, partial_rotary_factor=0.5))
    assert cos.shape == (64, 8) and torch.equal(cos, plain.rope_tables(1e4, 16, 64)[0])
    g = torch.Generator().manual_seed(2)
    x = torch.randn(3, 2, 32, generator=g, dtype=torch.float64)
    out = plain.apply_rope(x, torch.tensor([5, 9, 60]), cos.double(), sin.double())
    assert torch.equal(out[..., 16:], x[..., 16:]) and not torch.allclose(out[..., :16], x[..., :16])
    assert torch.allclose(out[..., :8] ** 2 + out[..., 8:16] ** 2, x[..., :8] ** 2 + x[..., 8:16] ** 2)
    pm = _tiny_weights("Y", tmp_path)
    ids = [5, 77, 200, 41, 9, 150, 123, 8]
    assert torch.allclose(pm.logits(ids), plain.model_logits(pm.config, pm.weights, ids, start=140), atol=2e-4)
    assert plain.scaled_rope_tables(pm.config)[0].shape == (160, 8)


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


# ---- q/k norm and the embedding's scale -----------------------------------------------------------
def _attention_inputs(tmp_path, T=7, eps=None):
    """Tiny A's layer 0 in float64 (4 query heads in 2 groups, head size 32) with q_norm and k_norm
    weights that differ within every rotation pair (i, i + d/2)."""
    pm = _tiny_weights("A", tmp_path)
    c = dict(pm.config)
    if eps is not None:
        c["rms_norm_eps"] = eps
    p = "model.layers.0.self_attn"
    W = {k: v.double().clone() for k, v in pm.weights.items() if k.startswith(p)}
    d = c["head_dim"]
    g = torch.Generator().manual_seed(12)
    W[f"{p}.q_norm.weight"] = 0.5 + torch.rand(d, generator=g, dtype=torch.float64) * 2.0
    W[f"{p}.k_norm.weight"] = 0.5 + torch.rand(d, generator=g, dtype=torch.float64) * 2.0
    x = torch.randn(T, c["hidden_size"], generator=g, dtype=torch.float64)
    positions = torch.arange(5, 5 + T)
    cos, sin = plain.rope_tables(c["rope_theta"], d, 64)
    return c, W, p, x, positions, cos.double(), sin.double()


def test_qk_norm_is_per_head_with_one_weight_for_all_heads(tmp_path):
    """The norm runs on [T * heads, d] with one weight vector of d values
    (/root/reference/src/models/layers/attention.rs:732-741): (1) permuting the query heads together
    with their kv heads, and the columns of o_proj with them, leaves the block's output unchanged (a
    weight per head would not); (2) with eps = 0, multiplying one head's rows of q_proj, or one kv
    head's rows of k_proj, by a constant changes nothing (a norm over all heads together, the full-width
    form of attention.rs:723-731, would let it through to the other heads)."""
    c, W, p, x, positions, cos, sin = _attention_inputs(tmp_path, eps=0.0)
    nq, nkv, d = c["num_attention_heads"], c["num_key_value_heads"], c["head_dim"]
    base = plain.attention_block(x, W, p, c, positions, cos, sin, None)

    def heads(w, n, order):                    # rows of a projection, head blocks reordered
        return w.reshape(n, d, -1)[order].reshape(n * d, -1)
    q_order, kv_order = [2, 3, 0, 1], [1, 0]   # the two groups change places
    W2 = dict(W)
    W2[f"{p}.q_proj.weight"] = heads(W[f"{p}.q_proj.weight"], nq, q_order)
    W2[f"{p}.k_proj.weight"] = heads(W[f"{p}.k_proj.weight"], nkv, kv_order)
    W2[f"{p}.v_proj.weight"] = heads(W[f"{p}.v_proj.weight"], nkv, kv_order)
    W2[f"{p}.o_proj.weight"] = heads(W[f"{p}.o_proj.weight"].T.contiguous(), nq, q_order).T
    assert torch.allclose(plain.attention_block(x, W2, p, c, positions, cos, sin, None), base, atol=1e-12)
    # within a group the query heads may change places too, the kv heads staying
    W3 = dict(W)
    W3[f"{p}.q_proj.weight"] = heads(W[f"{p}.q_proj.weight"], nq, [1, 0, 2, 3])
    W3[f"{p}.o_proj.weight"] = heads(W[f"{p}.o_proj.weight"].T.contiguous(), nq, [1, 0, 2, 3]).T
    assert torch.allclose(plain.attention_block(x, W3, p, c, positions, cos, sin, None), base, atol=1e-12)

    W4 = dict(W)
    wq = W[f"{p}.q_proj.weight"].clone()
    wq[d:2 * d] *= 7.0                          # query head 1 alone
    wk = W[f"{p}.k_proj.weight"].clone()
    wk[:d] *= 0.2                               # kv head 0 alone
    W4[f"{p}.q_proj.weight"], W4[f"{p}.k_proj.weight"] = wq, wk
    assert torch.allclose(plain.attention_block(x, W4, p, c, positions, cos, sin, None), base, atol=1e-10)
    # ... while the same constant on v does change the output: the norm is on q and k alone
    W5 = dict(W)
    W5[f"{p}.v_proj.weight"] = W[f"{p}.v_proj.weight"] * 2.0
    assert not torch.allclose(plain.attention_block(x, W5, p, c, positions, cos, sin, None), base, atol=1e-3)


def test_qk_norm_runs_before_the_rotation_and_adds_no_one(tmp_path):
    """The block must equal its parts put together in the reference's order: projections, per-head
    norm with the plain weight (no 1 + w: qk_norm_add_one is false for Qwen3, attention.rs:491),
    rotation (attention.rs:868-879, after prepare_qk_for_rope), attention, o_proj.  With weights that
    differ within a rotation pair the other order (rotate, then norm) gives another result, and
    so does 1 + w."""
    c, W, p, x, positions, cos, sin = _attention_inputs(tmp_path)
    T, nq, nkv, d, eps = x.shape[0], c["num_attention_heads"], c["num_key_value_heads"], c["head_dim"], c["rms_norm_eps"]
    q = (x @ W[f"{p}.q_proj.weight"].T).reshape(T, nq, d)
    k = (x @ W[f"{p}.k_proj.weight"].T).reshape(T, nkv, d)
    v = (x @ W[f"{p}.v_proj.weight"].T).reshape(T, nkv, d)
    wq, wk = W[f"{p}.q_norm.weight"], W[f"{p}.k_norm.weight"]
    rope = lambda t: plain.apply_rope(t, positions, cos, sin)
    out = lambda qq, kk: plain.attention(qq, kk, v).reshape(T, nq * d) @ W[f"{p}.o_proj.weight"].T
    norm_then_rotate = out(rope(plain.rms_norm(q, wq, eps)), rope(plain.rms_norm(k, wk, eps)))
    rotate_then_norm = out(plain.rms_norm(rope(q), wq, eps), plain.rms_norm(rope(k), wk, eps))
    plus_one = out(rope(plain.rms_norm(q, 1.0 + wq, eps)), rope(plain.rms_norm(k, 1.0 + wk, eps)))
    no_norm = out(rope(q), rope(k))
    got = plain.attention_block(x, W, p, c, positions, cos, sin, None)
    assert torch.allclose(got, norm_then_rotate, atol=1e-13)
    scale = float(got.abs().max())
    for other in (rotate_then_norm, plus_one, no_norm):
        assert float((got - other).abs().max()) > 1e-2 * scale
    # the sum of squares of a row survives the rotation, so with a constant weight the two orders agree:
    # only the place of the weight tells them apart
    ones = torch.ones(d, dtype=torch.float64)
    assert torch.allclose(rope(plain.rms_norm(q, ones, eps)), plain.rms_norm(rope(q), ones, eps), atol=1e-12)


def test_embedding_is_not_scaled(tmp_path):
    """x = E[ids] goes into the stream as it is (/root/reference/src/models/qwen3.rs:302-309): a
    one-layer model's logits equal the parts put together on the bare table rows, and a table
    multiplied by a constant (what a hidden sqrt(hidden_size) would amount to) gives other logits:
    the first norm removes the scale from the branches, but not from the residual path."""
    pm = _tiny_weights("B", tmp_path)                          # untied head
    c = dict(pm.config, num_hidden_layers=1)
    W = pm.weights
    ids = [4, 99, 310, 7, 250]
    cos, sin = plain.rope_tables(float(c["rope_theta"]), c["head_dim"], c["max_position_embeddings"])
    x = W["model.embed_tokens.weight"][torch.tensor(ids)]
    y = plain.decoder_layer(x, W, 0, c, torch.arange(len(ids)), cos.double(), sin.double())
    want = plain.rms_norm(y, W["model.norm.weight"], c["rms_norm_eps"]) @ W["lm_head.weight"].T
    got = plain.model_logits(c, W, ids)
    assert torch.allclose(got.double(), want, atol=1e-5)
    for factor in (math.sqrt(c["hidden_size"]), 1.0 / math.sqrt(c["hidden_size"])):
        W2 = dict(W)
        W2["model.embed_tokens.weight"] = W["model.embed_tokens.weight"] * factor
        other = plain.model_logits(c, W2, ids)
        assert float((other - got).abs().max()) > 1e-2 * float(got.abs().max())
