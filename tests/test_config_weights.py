"""Configuration, registry, weight loading errors, random-weights folders (no GPU)."""
import json
import os

import pytest
import torch

from configs import TINY
from xinfer_amd.config import ConfigError, Qwen3Config
from xinfer_amd.engine.model import CausalLM
from xinfer_amd.models import config_from_dict, family_of, load_config, registered_architectures
from xinfer_amd.weights import (RandomStore, SafetensorsStore, WeightError, write_random_model,
                                write_safetensors)


def test_both_tiny_configs_round_trip(tmp_path):
    for name, t in TINY.items():
        fam, cfg = config_from_dict(t["config"])
        assert isinstance(cfg, Qwen3Config)
        d = tmp_path / name
        d.mkdir()
        (d / "config.json").write_text(json.dumps(cfg.to_dict()))
        fam2, cfg2 = load_config(str(d))
        assert cfg2 == cfg and fam2 is fam
        for key in ("hidden_size", "num_attention_heads", "num_key_value_heads", "head_dim", "vocab_size",
                    "intermediate_size", "num_hidden_layers", "rms_norm_eps", "rope_theta",
                    "max_position_embeddings", "tie_word_embeddings"):
            assert getattr(cfg, key) == t["config"][key], key


def test_defaults_follow_the_reference():
    raw = dict(TINY["A"]["config"])
    for k in ("head_dim", "rope_theta", "tie_word_embeddings"):
        raw.pop(k)
    _, cfg = config_from_dict(raw)
    assert cfg.head_dim == 64 // 4          # hidden / heads (attention.rs:446)
    assert cfg.rope_theta == 10000.0        # rotary_emb.rs:49
    assert cfg.tie_word_embeddings is False


@pytest.mark.parametrize("change,needle", [
    (dict(num_key_value_heads=3), "multiple"),
    (dict(head_dim=15), "even"),
    (dict(hidden_act="gelu"), "hidden_act"),
    (dict(rope_scaling={"rope_type": "su", "factor": 4.0}), "Unknown rope_type: su"),
    (dict(rope_scaling={"rope_type": "yarn"}), "yarn rope_type requires factor"),
    (dict(rope_scaling={"type": "linear"}), "Linear rope_type requires factor"),
    (dict(rope_scaling={"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0}), "Llama3 rope_type requires"),
    (dict(rope_scaling={"rope_type": "dynamic"}), "Dynamic rope_type requires either alpha or factor"),
    (dict(rope_scaling={"rope_type": "yarn", "factor": "4"}), "rope_scaling.factor"),
    (dict(rope_scaling={"rope_type": "yarn", "factor": -1.0}), "positive"),
    (dict(rope_scaling=[1, 2]), "rope_scaling"),
    (dict(partial_rotary_factor=1.5), "partial_rotary_factor"),
    (dict(attn_logit_softcapping=30.0), "attn_logit_softcapping"),
    (dict(attn_output_gate=True), "attn_output_gate"),
    (dict(partial_rotary_factor=0.1), "even number"),
    (dict(sliding_window=0), "sliding_window"),
    (dict(layer_types=["full_attention"]), "layer_types"),
    (dict(hidden_size="64"), "integer"),
    (dict(vocab_size=None), "vocab_size"),
])
def test_bad_configs_are_refused(change, needle):
    raw = dict(TINY["A"]["config"], **change)
    with pytest.raises(ConfigError, match=needle):
        config_from_dict(raw)


def test_missing_required_key():
    raw = dict(TINY["A"]["config"])
    raw.pop("num_hidden_layers")
    with pytest.raises(ConfigError, match="num_hidden_layers"):
        config_from_dict(raw)


def test_registry():
    assert "Qwen3ForCausalLM" in registered_architectures()
    with pytest.raises(ConfigError, match="Unsupported architecture"):
        family_of("NoSuchModelForCausalLM")
    with pytest.raises(ConfigError, match="exactly one"):
        config_from_dict(dict(TINY["A"]["config"], architectures=["A", "B"]))


def test_window_per_layer():
    _, cfg = config_from_dict(TINY["W"]["config"])
    assert [cfg.window_of_layer(i) for i in range(3)] == [24, None, 24]
    spec = family_of(cfg.architecture).build_spec(cfg)
    m = CausalLM(spec, torch.float32)
    assert [(g.window, g.layers) for g in m.cache_groups] == [(24, (0, 2)), (0, (1,))]
    # without layer_types the window applies to every layer, as the reference passes it on
    raw = dict(TINY["W"]["config"])
    raw.pop("layer_types")
    _, cfg = config_from_dict(raw)
    assert [cfg.window_of_layer(i) for i in range(3)] == [24, 24, 24]


def test_no_size_stands_in_code():
    """The spec carries every size from the config; two configs give different specs."""
    specs = []
    for name in ("A", "B"):
        fam, cfg = config_from_dict(TINY[name]["config"])
        specs.append(fam.build_spec(cfg))
    a, b = specs
    assert a.layers[0].mixer.params != b.layers[0].mixer.params
    assert a.head["name"] == "model.embed_tokens.weight" and b.head["name"] == "lm_head.weight"


def _decls(name):
    fam, cfg = config_from_dict(TINY[name]["config"])
    return CausalLM.declare(fam.build_spec(cfg))


def test_random_folder_round_trip(tmp_path):
    d = write_random_model(str(tmp_path / "m"), TINY["B"]["config"], seed=1, linear_std=0.03, norm_std=0.05)
    assert sorted(os.listdir(d)) == ["config.json", "model.safetensors"]
    st = SafetensorsStore(d)
    decls = _decls("B")
    st.check(decls)
    assert {x.name for x in decls} == set(st.names())
    w = st.get("model.layers.2.mlp.down_proj.weight")
    assert w.dtype == torch.bfloat16 and tuple(w.shape) == (96, 224)
    assert abs(float(w.float().std()) - 0.03) < 0.003
    n = st.get("model.layers.0.self_attn.k_norm.weight").float()
    assert abs(float(n.mean()) - 1.0) < 0.05
    # same seed, same values; another seed, other values; a tensor does not depend on the others
    rs = RandomStore(decls, 1, 0.03, 0.05)
    assert torch.equal(rs.get("model.layers.2.mlp.down_proj.weight"), w)
    assert not torch.equal(RandomStore(decls, 2, 0.03, 0.05).get("model.layers.2.mlp.down_proj.weight"), w)
    one = RandomStore([x for x in decls if x.name == "model.layers.2.mlp.down_proj.weight"], 1, 0.03, 0.05)
    assert torch.equal(one.get("model.layers.2.mlp.down_proj.weight"), w)
    # the plain implementation's reader sees the same bytes
    from safetensors import safe_open
    with safe_open(os.path.join(d, "model.safetensors"), framework="pt") as f:
        assert torch.equal(f.get_tensor("model.layers.2.mlp.down_proj.weight"), w)


def test_counter_normal_values_depend_on_key_and_index_alone():
    """The CPU half of the random weights: a value is a function of (key, index), whatever the
    piece it is made in; the values are normal (moments, tails, a Kolmogorov-Smirnov distance)
    and two keys share nothing."""
    import numpy as np
    from xinfer_amd.weights.counter_normal import counter_normal
    x = counter_normal(0x1234_5678_9ABC_DEF0, 0, 300_000)
    assert x.dtype == np.float32 and np.isfinite(x).all()
    assert np.array_equal(counter_normal(0x1234_5678_9ABC_DEF0, 65_530, 70_001), x[65_530:135_531])
    assert abs(float(x.mean())) < 0.01 and abs(float(x.std()) - 1.0) < 0.01
    assert abs(float((np.abs(x) < 0.6745).mean()) - 0.5) < 0.005 and abs(float((x > 2).mean()) - 0.02275) < 0.002
    grid = np.sort(x.astype(np.float64))
    from math import erf, sqrt
    cdf = np.array([0.5 * (1 + erf(v / sqrt(2))) for v in grid[::100]])
    assert float(np.abs(cdf - np.arange(0, grid.size, 100) / grid.size).max()) < 0.005
    y = counter_normal(0x1234_5678_9ABC_DEF1, 0, 300_000)
    assert abs(float(np.corrcoef(x, y)[0, 1])) < 0.01 and abs(float(np.corrcoef(x[:-1], x[1:])[0, 1])) < 0.01
    z = counter_normal(7, 5, 1000, scale=0.02, shift=1.0)
    assert np.array_equal(z, counter_normal(7, 5, 1000) * np.float32(0.02) + np.float32(1.0))


def test_one_error_lists_everything_wrong(tmp_path):
    d = write_random_model(str(tmp_path / "m"), TINY["A"]["config"], seed=0)
    st = SafetensorsStore(d)
    tensors = {n: st.get(n) for n in st.names()}
    del tensors["model.layers.1.self_attn.q_norm.weight"]
    del tensors["model.norm.weight"]
    tensors["model.layers.0.mlp.gate_proj.weight"] = torch.zeros(128, 63, dtype=torch.bfloat16)
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(16)
    bad = tmp_path / "bad"
    bad.mkdir()
    write_safetensors(str(bad / "model.safetensors"), tensors.items())
    with pytest.raises(WeightError) as e:
        SafetensorsStore(str(bad)).check(_decls("A"))
    err = e.value
    assert err.missing == ["model.layers.1.self_attn.q_norm.weight", "model.norm.weight"]
    assert err.unexpected == ["model.layers.0.self_attn.rotary_emb.inv_freq"]
    assert err.wrong_shape == [("model.layers.0.mlp.gate_proj.weight", (128, 63), (128, 64))]
    text = str(err)
    for needle in ("missing", "unexpected", "wrong shapes", "q_norm", "inv_freq", "[128, 63]", "[128, 64]"):
        assert needle in text


def test_tensors_nobody_asks_for_are_ignored(tmp_path, capfd):
    """The reference reads by name and never looks at the rest: a tied checkpoint that also stores
    lm_head.weight, or an old export's rotary_emb.inv_freq, loads, and the head is the embedding
    table (/root/reference/src/models/qwen3.rs:267-287).  `check` returns the ignored names and the
    loader says so once."""
    from xinfer_amd.engine.loading import build_model
    d = write_random_model(str(tmp_path / "m"), TINY["A"]["config"], seed=0)
    st = SafetensorsStore(d)
    assert "lm_head.weight" not in st.names()
    tensors = {n: st.get(n) for n in st.names()}
    tensors["lm_head.weight"] = torch.full_like(tensors["model.embed_tokens.weight"], 3.0)    # not the table's values
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(16)
    extra = tmp_path / "extra"
    extra.mkdir()
    write_safetensors(str(extra / "model.safetensors"), tensors.items())
    store = SafetensorsStore(str(extra))
    assert store.check(_decls("A")) == ["lm_head.weight", "model.layers.0.self_attn.rotary_emb.inv_freq"]
    _, cfg = config_from_dict(TINY["A"]["config"])
    model = build_model(cfg, store, "f32", device="cpu")
    assert model.ignored_tensors == ["lm_head.weight", "model.layers.0.self_attn.rotary_emb.inv_freq"]
    assert model.head.tied and model.head.proj.weight.data_ptr() == model.embedding.table.data_ptr()
    assert "2 tensors the model does not use are ignored" in capfd.readouterr().err
    # a missing tensor is still the one error, and it lists the ignored ones beside it
    del tensors["model.norm.weight"]
    bad = tmp_path / "bad"
    bad.mkdir()
    write_safetensors(str(bad / "model.safetensors"), tensors.items())
    with pytest.raises(WeightError) as e:
        SafetensorsStore(str(bad)).check(_decls("A"))
    assert e.value.missing == ["model.norm.weight"] and "lm_head.weight" in e.value.unexpected


def test_checkpoint_without_the_model_prefix_is_tied(tmp_path):
    """A checkpoint that holds embed_tokens.weight without the `model.` prefix: every tensor is read
    without the prefix and the head is the table, whatever config.json says about tying
    (/root/reference/src/models/qwen3.rs:200-209)."""
    from xinfer_amd.engine.loading import build_model
    raw = dict(TINY["B"]["config"])
    assert raw["tie_word_embeddings"] is False
    d = write_random_model(str(tmp_path / "m"), raw, seed=1)
    st = SafetensorsStore(d)
    tensors = {n[len("model."):]: st.get(n) for n in st.names() if n.startswith("model.")}
    bare = tmp_path / "bare"
    bare.mkdir()
    write_safetensors(str(bare / "model.safetensors"), tensors.items())
    _, cfg = config_from_dict(raw)
    store = SafetensorsStore(str(bare))
    model = build_model(cfg, store, "f32", device="cpu")
    assert model.spec.layers[0].prefix == "layers.0" and model.head.tied and model.ignored_tensors == []
    assert torch.equal(model.embedding.table, tensors["embed_tokens.weight"].float())
    assert model.head.proj.weight.data_ptr() == model.embedding.table.data_ptr()
    assert torch.equal(model.final_norm.weight, tensors["norm.weight"].float())
    # with the prefix the same config is untied
    assert not build_model(cfg, st, "f32", device="cpu").head.tied


def test_storage_policy(tmp_path):
    """bfloat16 stays, float16 becomes bfloat16, a tensor stored in 32 bits stays in 32 bits,
    integer tables become int32."""
    path = str(tmp_path / "model.safetensors")
    write_safetensors(path, [("a", torch.ones(3, dtype=torch.bfloat16)), ("b", torch.ones(3, dtype=torch.float16)),
                             ("c", torch.full((3,), 1.0000001, dtype=torch.float32)),
                             ("d", torch.arange(3, dtype=torch.int64)), ("e", torch.ones(2, dtype=torch.float64))])
    st = SafetensorsStore(str(tmp_path))
    assert st.get("a").dtype == torch.bfloat16
    assert st.get("b").dtype == torch.bfloat16
    assert st.get("c").dtype == torch.float32 and float(st.get("c")[0]) == float(torch.tensor(1.0000001))
    assert st.get("d").dtype == torch.int32
    assert st.get("e").dtype == torch.bfloat16
    assert st.get("a", torch.float32).dtype == torch.float32


def test_no_weight_files(tmp_path):
    with pytest.raises(FileNotFoundError, match="No weight files"):
        SafetensorsStore(str(tmp_path))
    with pytest.raises(ConfigError, match="config.json"):
        load_config(str(tmp_path))


def test_command_line_options_follow_the_reference():
    """Names and defaults of /root/reference/src/server/mod.rs:706-904 for the options that
    have a part here."""
    from xinfer_amd.cli import build_parser
    a = build_parser().parse_args([])
    assert (a.m, a.w, a.dtype, a.max_num_seqs, a.max_tokens, a.prefill_chunk_size) == (None, None, "bf16", 1, 16384, 8192)
    assert a.max_model_len is None and a.temperature is None and a.top_k is None and a.top_p is None
    assert not a.ignore_eos and not a.disable_cuda_graph and a.seed is None and a.batch is None and not a.interactive
    assert build_parser().parse_args(["--i"]).interactive
    a = build_parser().parse_args(["--m", "x", "--prompts", "a|b", "--max-num-seqs", "4", "--top-k", "5", "--top-p", "0.9",
                                   "--temperature", "0.5", "--kv-fraction", "0.3", "--disable-cuda-graph"])
    assert a.prompts == "a|b" and a.max_num_seqs == 4 and a.top_k == 5 and a.kv_fraction == 0.3 and a.disable_cuda_graph


def test_bench_refuses_more_than_one_gpu():
    """The measurement script runs on one GPU: for more it prints one line that says so and
    exits with 2, before anything touches a GPU."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode == 2
    lines = [l for l in r.stdout.splitlines() if l.strip()]
    assert len(lines) == 1 and "one GPU" in lines[0]


# ---- rope scaling ----------------------------------------------------------------------------
ROPE_SCALINGS = [
    (dict(rope_type="yarn", factor=4.0, original_max_position_embeddings=32), None),
    (dict(type="yarn", factor=8.0, beta_fast=16, beta_slow=2, attn_factor=1.3, extrapolation_factor=0.9), 0.5),
    (dict(rope_type="linear", factor=3.0), None),
    (dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0, original_max_position_embeddings=16), None),
    (dict(rope_type="dynamic", factor=2.5), 0.75),
    (dict(rope_type="dynamic", alpha=3.0), None),
    (dict(rope_type="default"), None),
    (None, 0.25),
]


@pytest.mark.parametrize("scaling,partial", ROPE_SCALINGS)
def test_rope_scaling_tables_are_the_plain_ones(scaling, partial):
    """The position encoding part alone, on the CPU: for every kind of rope_scaling and a partial
    rotation its tables equal the plain implementation's, which is written from the reference
    on its own (tests/plain_qwen3.py: scaled_rope_tables), and the model's positions are the
    table's rows."""
    import torch
    import plain_qwen3 as plain
    from xinfer_amd.parts import position_encoding_class
    raw = dict(TINY["A"]["config"], max_position_embeddings=128)
    if scaling is not None:
        raw["rope_scaling"] = scaling
    if partial is not None:
        raw["partial_rotary_factor"] = partial
    fam, cfg = config_from_dict(raw)
    spec = fam.build_spec(cfg)
    pe = spec.layers[0].mixer["position"]
    part = position_encoding_class(pe.kind)(pe, torch.float32)
    part.load(None, "", "cpu")
    cos, sin = plain.scaled_rope_tables(dict(raw))
    assert part.cos.shape == cos.shape == (spec.max_positions, int((partial or 1.0) * 32) // 2)
    assert torch.equal(part.cos, cos) and torch.equal(part.sin, sin)
    assert part.rotary_dim == 2 * cos.shape[1] and part.head_dim == 32
    # the configuration survives being written out and read again
    assert config_from_dict(cfg.to_dict())[1] == cfg


def test_yarn_scaling_factor_option():
    """The option puts YaRN over the file's own length in place of whatever the file says, with the
    derived parameters of /root/reference/src/utils/mod.rs:806-871: beta_fast 32 up to a factor of
    4 and 32 sqrt(factor / 4) beyond, the extrapolation factor 1 + 0.05 sqrt(factor - 8) above 8;
    the model then runs round(length * factor) positions."""
    from xinfer_amd.config.model_config import derive_yarn_scaling
    _, cfg = config_from_dict(dict(TINY["A"]["config"], rope_scaling=dict(rope_type="linear", factor=2.0)))
    assert cfg.positions == 128
    y = cfg.with_yarn_scaling(4.0)
    rs = y.rope_scaling
    assert (rs.kind, rs.factor, rs.original_max_position_embeddings, rs.beta_fast, rs.beta_slow,
            rs.extrapolation_factor, rs.attn_factor) == ("yarn", 4.0, 128.0, 32.0, 1.0, 1.0, 1.0)
    assert y.positions == 512 and y.max_position_embeddings == 128
    big = derive_yarn_scaling(16.0, 4096)
    assert big.beta_fast == 64.0 and abs(big.extrapolation_factor - (1 + 0.05 * 8 ** 0.5)) < 1e-12
    assert derive_yarn_scaling(0.5, 4096).factor == 1.0          # a factor below 1 is 1


def test_biases_follow_the_checkpoint_when_the_config_is_silent(tmp_path):
    """`qkv_bias` goes before `attention_bias`; with neither key the q, k and v biases are taken if
    the checkpoint has them (/root/reference/src/models/layers/attention.rs:472-476, 388-399): the
    same tensors give a model with biases under a config.json without the key, one without them
    (and three ignored tensors a layer) when the key says false."""
    from xinfer_amd.engine.loading import build_model
    raw = dict(TINY["W"]["config"])
    assert raw["attention_bias"] is True
    d = write_random_model(str(tmp_path / "w"), raw, seed=2)
    store = SafetensorsStore(d)
    silent = {k: v for k, v in raw.items() if k != "attention_bias"}
    fam, cfg = config_from_dict(silent)
    assert cfg.attention_bias is None
    assert fam.spec(cfg, store.names()).layers[0].mixer["bias"] is True
    assert fam.spec(cfg, [n for n in store.names() if not n.endswith(".bias")]).layers[0].mixer["bias"] is False
    assert fam.build_spec(cfg).layers[0].mixer["bias"] is False                     # random weights: none
    assert config_from_dict(dict(silent, qkv_bias=True, attention_bias=False))[1].attention_bias is True
    assert config_from_dict(dict(silent, qkv_bias=False, attention_bias=True))[1].attention_bias is False
    with_bias = build_model(cfg, store, "f32", device="cpu")
    assert with_bias.ignored_tensors == [] and with_bias.blocks[0].mixer.qkv_bias is not None
    _, off = config_from_dict(dict(silent, attention_bias=False))
    without = build_model(off, store, "f32", device="cpu")
    assert len(without.ignored_tensors) == 3 * raw["num_hidden_layers"] and without.blocks[0].mixer.qkv_bias is None
