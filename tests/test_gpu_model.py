"""The engine against the plain implementation, in float32 and in bfloat16, under every way
of cutting the work: whole requests; most of a request in one step and its last 32 tokens
one by one; portions of changing size down to two tokens; and mixed batches of up to four
live requests with so few pages that pages are used again."""
import random

import pytest
import torch

import harness
import plain_qwen3 as plain
from configs import REAL, TINY

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]
LENGTHS = {"A": [5, 17, 33, 100, 128], "B": [1, 9, 64, 130, 200], "W": [3, 24, 25, 77, 150, 61],
           "O": [2, 31, 70, 129, 8], "Y": [4, 64, 65, 160, 41, 100]}


def _requests(name):
    rng = random.Random(100 + ord(name))
    vocab = TINY[name]["config"]["vocab_size"]
    return {f"r{i}": harness.random_prompt(rng, n, vocab) for i, n in enumerate(LENGTHS[name])}


_plain_cache = {}


def _plain_logits(name, model_dir):
    if name not in _plain_cache:
        pm = plain.PlainModel(model_dir)
        _plain_cache[name] = {rid: pm.logits(toks) for rid, toks in _requests(name).items()}
    return _plain_cache[name]


_runner_cache = {}


def _runner(name, dtype, model_dir, num_pages):
    """One loaded model per (config, dtype); a fresh runner (and so a fresh cache) per test."""
    from xinfer_amd.engine import ModelRunner, load_model
    key = (name, dtype)
    if key not in _runner_cache:
        _runner_cache[key] = load_model(model_dir, dtype, "cuda:0")
    return ModelRunner(_runner_cache[key], page_size=TINY[name]["page_size"], num_pages=num_pages,
                       max_requests=4)


def _run(name, dtype, model_dirs, steps, what):
    page = TINY[name]["page_size"]
    need = harness.tokens_needed(steps, page)
    runner = _runner(name, dtype, model_dirs[name], need // page)       # exactly enough pages
    got = harness.replay(runner, steps)
    for g in range(len(runner.cache.groups)):
        assert runner.cache.free_pages(g) == need // page               # every page came back
    ref = _plain_logits(name, model_dirs[name])
    rel = harness.compare(got, ref, harness.TOL[dtype], f"{name}/{dtype}/{what}")
    print(f"{name}/{dtype}/{what}: worst error {rel:.2e} of the largest logit")
    return got


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(TINY))
def test_whole(name, dtype, model_dirs):
    got = _run(name, dtype, model_dirs, harness.trace_whole(_requests(name)), "whole")
    assert len(got) == sum(LENGTHS[name])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(TINY))
def test_tail_one_by_one(name, dtype, model_dirs):
    _run(name, dtype, model_dirs, harness.trace_tail_one_by_one(_requests(name)), "tail")


@pytest.mark.parametrize("name", list(TINY))
def test_decode_steps_with_the_attention_kernel_doing_the_steps_own_work(name, model_dirs):
    """Steps of single tokens in bfloat16 let the attention kernel norm and rotate its heads and
    store the new keys and values; with that switched off (the kernel of its own before the
    attention, as in steps that bring portions) the logits are the same bit for bit."""
    from xinfer_amd.engine import load_model
    from xinfer_amd import kernels
    together = dict([(k, v) for k, v in _requests(name).items() if len(v) > 8][:4])
    steps = harness.trace_tail_one_by_one(_requests(name)) + harness.trace_batch_decode(together, tail=6)
    _run(name, "bfloat16", model_dirs, steps, "tail")                 # warms the cached model too
    model = _runner_cache[(name, "bfloat16")]
    mixers = [b.mixer for b in model.blocks]
    assert all(m.decode_packed for m in mixers)
    calls = []
    inner = kernels.attention_decode_packed_bf16
    kernels.attention_decode_packed_bf16 = lambda *a, **k: (calls.append(1), inner(*a, **k))[1]
    try:
        got = _run(name, "bfloat16", model_dirs, steps, "tail, packed")
        assert calls
        for m in mixers:
            m.decode_packed = False
        n = len(calls)
        again = _run(name, "bfloat16", model_dirs, steps, "tail, two kernels")
        assert len(calls) == n
    finally:
        kernels.attention_decode_packed_bf16 = inner
        for m in mixers:
            m.decode_packed = True
    assert got.keys() == again.keys() and all(torch.equal(got[k], again[k]) for k in got)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(TINY))
def test_portions(name, dtype, model_dirs):
    _run(name, dtype, model_dirs, harness.trace_portions(_requests(name)), "portions")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(TINY))
@pytest.mark.parametrize("seed", [0, 1])
def test_mixed(name, dtype, seed, model_dirs):
    reqs = _requests(name)
    steps = harness.trace_mixed(reqs, seed)
    page = TINY[name]["page_size"]
    # fewer pages than all requests together would need: later requests reuse pages
    assert harness.tokens_needed(steps, page) < sum(-(-len(t) // page) * page for t in reqs.values())
    _run(name, dtype, model_dirs, steps, f"mixed{seed}")


@pytest.mark.parametrize("name", list(TINY))
def test_float32_does_not_depend_on_cutting(name, model_dirs):
    """In float32 every reduction's order is fixed by the position alone, so logits are
    bit-equal however the tokens were cut and batched."""
    reqs = _requests(name)
    a = _run(name, "float32", model_dirs, harness.trace_whole(reqs), "whole")
    b = _run(name, "float32", model_dirs, harness.trace_mixed(reqs, 7), "mixed7")
    c = _run(name, "float32", model_dirs, harness.trace_portions(reqs), "portions")
    for key in a:
        assert torch.equal(a[key], b[key]), key
        assert torch.equal(a[key], c[key]), key


# ---- real layer sizes ---------------------------------------------------------------------------
@pytest.mark.parametrize("name", list(REAL))
def test_real_layer_sizes(name, real_model_dirs):
    """Qwen3-0.6B, 4B, 8B, 14B and 32B layer sizes (few layers, small vocabulary): whole requests, a
    mixed trace with pages used again and a tail decoded one by one, in float32 and in
    bfloat16, against the plain implementation."""
    from xinfer_amd.engine import ModelRunner, load_model
    t = REAL[name]
    d = real_model_dirs(name)
    vocab, page = t["config"]["vocab_size"], t["page_size"]
    rng = random.Random(5)
    reqs = {f"r{i}": harness.random_prompt(rng, n, vocab) for i, n in enumerate([70, 200, 129, 33])}
    pm = plain.PlainModel(d)
    ref = {rid: pm.logits(toks) for rid, toks in reqs.items()}
    del pm
    for dtype in DTYPES:
        model = load_model(d, dtype, "cuda:0")
        for what, steps in (("whole", harness.trace_whole(reqs)), ("mixed", harness.trace_mixed(reqs, 3, max_live=3)),
                            ("tail", harness.trace_tail_one_by_one(reqs, tail=8))):
            need = harness.tokens_needed(steps, page)
            runner = ModelRunner(model, page_size=page, num_pages=need // page, max_requests=4)
            got = harness.replay(runner, steps)
            rel = harness.compare(got, ref, harness.TOL[dtype], f"{name}/{dtype}/{what}")
            print(f"{name}/{dtype}/{what}: worst error {rel:.2e} of the largest logit")
            del runner
        del model
        torch.cuda.empty_cache()


@pytest.mark.parametrize("name,live", [("8B", 12), ("8B", 40), ("14B", 8), ("14B", 48), ("32B", 16), ("32B", 70), ("0.6B", 9), ("0.6B", 33),
                                       ("4B", 16), ("4B", 64), ("8B", 150), ("14B", 200), ("0.6B", 256), ("32B", 129)])
def test_real_layer_sizes_wide_decode_batches(name, live, real_model_dirs):
    """Decode steps of many requests at real layer sizes, in bfloat16: the kernels that serve 6 to
    16 rows (thin products with the folded norm, the gated tiled product), 17 to 64 (tiled
    products with partial sums), more (the library beside them) and 129 to 256 (the library's
    batched product over slices of K), inside the model against the plain implementation; the steps are launched one by one and, the third time on, replayed
    from a graph."""
    from xinfer_amd.engine import ModelRunner, load_model
    t = REAL[name]
    d = real_model_dirs(name)
    vocab, page = t["config"]["vocab_size"], t["page_size"]
    rng = random.Random(11)
    reqs = {f"r{i}": harness.random_prompt(rng, rng.randrange(8, 30), vocab) for i in range(live)}
    pm = plain.PlainModel(d)
    ref = {rid: pm.logits(toks) for rid, toks in reqs.items()}
    del pm
    model = load_model(d, "bfloat16", "cuda:0")
    steps = harness.trace_batch_decode(reqs, tail=5)
    runner = ModelRunner(model, page_size=page, num_pages=live + 2, max_requests=live, graph_after=3, graph_max_batch=64)
    got = harness.replay(runner, steps)
    rel = harness.compare(got, ref, harness.TOL["bfloat16"], f"{name}/bfloat16/decode batch of {live}")
    print(f"{name}/decode batch of {live}: worst error {rel:.2e} of the largest logit")
    assert (runner.graph_replays > 0) == (live <= 64)
    if live <= 64:      # the same steps launched one by one: the same logits to rounding (a replayed step
        del runner      # plans its kernels for the longest context of its bucket, so sums may be cut elsewhere)
        eager = ModelRunner(model, page_size=page, num_pages=live + 2, max_requests=live, use_graphs=False)
        again = harness.replay(eager, steps)
        harness.compare(again, ref, harness.TOL["bfloat16"], f"{name}/bfloat16/decode batch of {live}, launched")
        scale = max(float(r.abs().max()) for r in ref.values())
        assert max(float((got[k] - again[k]).abs().max()) for k in got) < 2e-3 * scale


def test_mixed_step_with_long_contexts_both_attention_paths(real_model_dirs):
    """A step that brings single tokens of six requests with contexts of some thousand tokens and a
    portion of a seventh, at Qwen3-8B layer sizes: the decode kernel takes the six (their contexts
    are long), the prefill kernel the portion; with the rule switched off the prefill kernel takes
    all.  The two agree to rounding, and a request alone gives the same logits as in the batch."""
    from xinfer_amd import kernels
    from xinfer_amd.engine import ModelRunner, StepEntry, load_model
    t = REAL["8B"]
    vocab, page = t["config"]["vocab_size"], t["page_size"]
    model = load_model(real_model_dirs("8B"), "bfloat16", "cuda:0")
    rng = random.Random(21)
    lens = [900, 1000, 700, 1003, 960, 1010]         # the model's 1,024 positions bound the contexts
    prompts = [harness.random_prompt(rng, n, vocab) for n in lens]
    portion = harness.random_prompt(rng, 300, vocab)
    nxt = [rng.randrange(vocab) for _ in lens]

    def run(switch_off):
        old = kernels.MIXED_DECODE_CONTEXT, kernels.MIXED_DECODE_WORK
        runner = ModelRunner(model, page_size=page, num_pages=8 * 16 + 8, max_requests=8, use_graphs=False)
        try:
            kernels.MIXED_DECODE_CONTEXT, kernels.MIXED_DECODE_WORK = (1 << 30, 1 << 60) if switch_off else (512, 1 << 60)
            for i, p in enumerate(prompts):
                runner.add_request(i)
                runner.step([StepEntry(i, p, [])])
            runner.add_request(7)
            entries = [StepEntry(i, [tok], [0]) for i, tok in enumerate(nxt)] + [StepEntry(7, portion, [0, 299])]
            return runner.step(entries).float().cpu()
        finally:
            kernels.MIXED_DECODE_CONTEXT, kernels.MIXED_DECODE_WORK = old

    split, together = run(False), run(True)
    scale = float(together.abs().max())
    assert float((split - together).abs().max()) < harness.TOL["bfloat16"] * scale
    assert not torch.equal(split[:6], together[:6])          # another kernel did run
    # the first request alone, decoded by the decode kernel as a batch of one
    runner = ModelRunner(model, page_size=page, num_pages=24, max_requests=2, use_graphs=False)
    runner.add_request(0)
    runner.step([StepEntry(0, prompts[0], [])])
    alone = runner.step([StepEntry(0, [nxt[0]], [0])]).float().cpu()
    assert float((alone[0] - split[0]).abs().max()) < harness.TOL["bfloat16"] * scale


def test_extra_tensors_and_a_checkpoint_without_prefix_give_the_same_logits(model_dirs, tmp_path):
    """A tied checkpoint that also stores an lm_head.weight (of other values) and a stray buffer
    gives the logits of the checkpoint without them: the head is the table.  A checkpoint whose
    names lack the `model.` prefix is read without it and tied (qwen3.rs:200-209): it gives the
    logits of the same tensors under the usual names with tie_word_embeddings set."""
    import json
    import shutil
    from xinfer_amd.engine import ModelRunner, StepEntry, load_model
    from xinfer_amd.weights import SafetensorsStore, write_safetensors
    toks = harness.random_prompt(random.Random(3), 40, 256)

    def logits(folder, page):
        runner = ModelRunner(load_model(folder, "float32", "cuda:0"), page_size=page, num_pages=8, max_requests=1)
        runner.add_request(0)
        return runner.step([StepEntry(0, toks, list(range(len(toks))))]).cpu()

    st = SafetensorsStore(model_dirs["A"])
    tensors = {n: st.get(n) for n in st.names()}
    tensors["lm_head.weight"] = torch.full_like(tensors["model.embed_tokens.weight"], 0.5)
    tensors["model.layers.1.self_attn.rotary_emb.inv_freq"] = torch.ones(16)
    extra = tmp_path / "extra"
    extra.mkdir()
    shutil.copy(model_dirs["A"] + "/config.json", extra / "config.json")
    write_safetensors(str(extra / "model.safetensors"), tensors.items())
    base = logits(model_dirs["A"], 16)
    assert torch.equal(logits(str(extra), 16), base)
    ref = plain.PlainModel(model_dirs["A"]).logits(toks)
    assert float((base - ref).abs().max()) < harness.TOL["float32"] * float(ref.abs().max())

    st = SafetensorsStore(model_dirs["B"])
    named = {n: st.get(n) for n in st.names() if n.startswith("model.")}
    with open(model_dirs["B"] + "/config.json") as f:
        raw = json.load(f)
    bare, tied = tmp_path / "bare", tmp_path / "tied"
    for folder, tens, cfg in ((bare, {n[len("model."):]: t for n, t in named.items()}, raw),
                              (tied, named, dict(raw, tie_word_embeddings=True))):
        folder.mkdir()
        (folder / "config.json").write_text(json.dumps(cfg))
        write_safetensors(str(folder / "model.safetensors"), tens.items())
    toks = [t % 509 for t in toks]
    assert torch.equal(logits(str(bare), 8), logits(str(tied), 8))
    ref = plain.PlainModel(str(tied)).logits(toks)
    assert float((logits(str(bare), 8) - ref).abs().max()) < harness.TOL["float32"] * float(ref.abs().max())


def test_a_config_that_is_silent_about_biases_takes_the_checkpoints(model_dirs, tmp_path):
    """Configuration W's folder with `attention_bias` taken out of config.json: the q, k and v
    biases in the checkpoint are used all the same (/root/reference/src/models/layers/attention.rs:
    472-476, 388-399), the logits are those of the folder that names them, and the plain model's."""
    import json
    import shutil
    from xinfer_amd.engine import ModelRunner, StepEntry, load_model
    toks = harness.random_prompt(random.Random(4), 50, 300)

    def logits(folder):
        runner = ModelRunner(load_model(folder, "float32", "cuda:0"), page_size=16, num_pages=[8, 8], max_requests=1)
        runner.add_request(0)
        return runner.step([StepEntry(0, toks, list(range(len(toks))))]).cpu()

    silent = tmp_path / "silent"
    silent.mkdir()
    with open(model_dirs["W"] + "/config.json") as f:
        raw = json.load(f)
    assert raw.pop("attention_bias") is True
    (silent / "config.json").write_text(json.dumps(raw))
    shutil.copy(model_dirs["W"] + "/model.safetensors", silent / "model.safetensors")
    got = logits(str(silent))
    assert torch.equal(got, logits(model_dirs["W"]))
    ref = plain.PlainModel(str(silent)).logits(toks)
    assert float((got - ref).abs().max()) < harness.TOL["float32"] * float(ref.abs().max())
    (silent / "config.json").write_text(json.dumps(dict(raw, qkv_bias=False)))
    assert not torch.allclose(logits(str(silent)), got, atol=1e-3)          # switched off, the biases are missed
