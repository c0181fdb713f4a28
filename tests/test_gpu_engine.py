"""Generation through the entry point, sampling kernels, the replay program, parts alone,
long decoding, and a toy mixer with state of its own registered from the test."""
import json
import os
import random
import subprocess
import sys

import numpy as np
import pytest
import torch

import harness
import plain_qwen3 as plain
import plain_sampling
from configs import TINY

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


# ---- sampling kernels ---------------------------------------------------------------------
def _logits(rows, V, seed, coarse=False):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(rows, V, generator=g) * 3
    if coarse:
        x = x.to(torch.bfloat16).float()          # many exact ties, as logits of a bfloat16 head have
    return x


@pytest.mark.parametrize("V", [256, 509, 151936])
def test_argmax_lowest_index_wins_ties(V):
    from xinfer_amd.sampling import Sampler
    s = Sampler(DEV)
    x = _logits(5, V, 1, coarse=True)
    x[2, 7] = x[2, V - 3] = 50.0
    out = s.argmax(x.to(DEV)).cpu()
    assert out.tolist() == [int(torch.nonzero(r == r.max())[0]) for r in x]
    assert out[2] == 7


@pytest.mark.parametrize("coarse", [False, True])
@pytest.mark.parametrize("V,T,k,p", [
    (256, 0.8, 0, 1.0), (509, 1.3, 0, 1.0), (300, 0.7, 32, 1.0), (300, 0.7, 0, 0.9),
    (300, 0.7, 32, 0.95), (2000, 1.0, 5, 0.5), (151936, 0.7, 32, 0.95), (151936, 1.0, 0, 0.8),
    (151936, 0.9, 64, 1.0), (151936, 0.7, 65, 0.95), (5000, 1.1, 1, 0.3), (163841, 0.8, 7, 0.6),
])
def test_sample_matches_plain(V, T, k, p, coarse):
    from xinfer_amd.sampling import Sampler, Strategy
    s = Sampler(DEV)
    rows = 6
    x = _logits(rows, V, 2, coarse)
    us = [0.0, 0.999999, 0.5, 0.123, 0.77, 0.31]
    got = s.sample(x.to(DEV).clone(), [Strategy(T, k, p)] * rows, us)
    for r in range(rows):
        kept = plain_sampling.kept_probabilities(x[r], T, k, p)
        want = plain_sampling.draw(kept, us[r])
        if got[r] != want:
            # float32 sums may put u on the other side of a boundary: then the two tokens are
            # neighbours among the kept ones and u lies within rounding of their boundary
            assert kept[got[r]] > 0, (r, got[r], want)
            cum = torch.cumsum(kept, 0) / kept.sum()
            lo, hi = sorted((got[r], want))
            assert float(kept[lo + 1:hi].sum()) == 0.0 and abs(float(cum[lo]) - us[r]) < 1e-5, (r, got[r], want)
        assert kept[got[r]] > 0


def test_sample_frequencies_follow_softmax():
    from xinfer_amd.sampling import Sampler, Strategy, uniform
    s = Sampler(DEV)
    V, n = 256, 4000
    x = _logits(1, V, 3)[0] * 0.5
    logits = x[None].repeat(n, 1).to(DEV)
    toks = s.sample(logits, [Strategy(0.8)] * n, [uniform(7, 0, i) for i in range(n)])
    freq = torch.bincount(torch.tensor(toks), minlength=V).double() / n
    want = torch.softmax(x.double() / 0.8, -1)
    assert float((freq - want).abs().sum()) < 0.25            # total variation of 4000 draws over 256 tokens
    assert abs(float(freq[want.argmax()]) - float(want.max())) < 0.03


def test_per_row_strategies_and_penalties():
    from xinfer_amd.sampling import Sampler, Strategy
    s = Sampler(DEV)
    V = 300
    x = _logits(3, V, 4)
    top = int(x[1].argmax())
    recent = [[], [top, top, 5], [9]]
    strat = [Strategy(), Strategy(0.0, frequency_penalty=100.0, presence_penalty=1.0), Strategy(0.9, 4, 1.0)]
    got = s.sample(x.to(DEV).clone(), strat, [0.1, 0.2, 0.3], recent=recent)
    assert got[0] == int(x[0].argmax())
    pen = plain_sampling.apply_penalties(x[1], recent[1], 100.0, 1.0)
    assert got[1] == int(pen.argmax()) != top
    assert got[2] == plain_sampling.draw(plain_sampling.kept_probabilities(x[2], 0.9, 4, 1.0), 0.3)


# ---- generation through the entry point ---------------------------------------------------------
def _engine(model_dir, name, dtype, **kw):
    from xinfer_amd import Engine, EngineConfig
    t = TINY[name]
    cfg = EngineConfig(weight_path=model_dir, page_size=t["page_size"], seed=5, **kw)
    return Engine(cfg, dtype)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_greedy_generation_tiny_a(dtype, model_dirs):
    """Workload of tiny configuration A: prompts of 5, 17 and 33 tokens, 16 greedy tokens each."""
    from xinfer_amd import SamplingParams
    rng = random.Random(0)
    prompts = [harness.random_prompt(rng, n, 256) for n in (5, 17, 33)]
    eng = _engine(model_dirs["A"], "A", dtype, max_num_seqs=4, num_pages=12, prefill_chunk_size=16)
    outs = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=16, ignore_eos=True))
    pm = plain.PlainModel(model_dirs["A"])
    for p, o in zip(prompts, outs):
        assert o.prompt_length == len(p) and o.decoded_length == 16 and o.finish_reason == "length"
        if dtype == "f32":
            assert o.token_ids == pm.greedy(p, 16)
        else:
            # bfloat16 may pick the other of two nearly equal logits; every token it picks must be
            # within tolerance of the plain maximum given the same history
            ids = list(p)
            for t in o.token_ids:
                lg = pm.logits(ids)[-1]
                assert float(lg.max() - lg[t]) <= 2 * harness.TOL["bfloat16"] * float(lg.abs().max())
                ids.append(t)
    assert eng.get_available_kv_tokens() == 12 * 16 and eng.runner.cache.live_requests() == 0


def test_tiny_b_workload_chunked_and_sampled(model_dirs):
    """Workload of tiny configuration B: prompts 1, 9, 64, 130, 200, chunk 48 mixed with decode,
    temperature 0.8 with a seed, 24 tokens each.  A request's tokens do not depend on what it was
    batched with: alone and together give the same tokens (float32)."""
    from xinfer_amd import SamplingParams
    rng = random.Random(1)
    prompts = [harness.random_prompt(rng, n, 509) for n in (1, 9, 64, 130, 200)]
    sps = [SamplingParams(temperature=0.8, max_tokens=24, ignore_eos=True, seed=100 + i) for i in range(5)]
    eng = _engine(model_dirs["B"], "B", "f32", max_num_seqs=4, num_pages=80, prefill_chunk_size=48,
                  max_num_batched_tokens=64)
    together = eng.generate(prompts, sps)
    assert [o.decoded_length for o in together] == [24] * 5
    assert len({tuple(o.token_ids) for o in together}) == 5
    eng2 = _engine(model_dirs["B"], "B", "f32", max_num_seqs=1, num_pages=40, prefill_chunk_size=1000)
    for i in (4, 0, 2):
        alone = eng2.generate([prompts[i]], sps[i])[0]             # the same seed, another request id
        assert alone.token_ids == together[i].token_ids, i
    # each token is the one the plain model draws at that point from its own logits with the same
    # uniform number (a request with a seed of its own draws from that seed's first stream)
    from xinfer_amd.sampling import uniform
    pm = plain.PlainModel(model_dirs["B"])
    for i in (1, 2):
        ids = list(prompts[i])
        for n, t in enumerate(together[i].token_ids):
            kept = plain_sampling.kept_probabilities(pm.logits(ids)[-1], 0.8)
            assert plain_sampling.draw(kept, uniform(100 + i, 0, n)) == t, (i, n)
            ids.append(t)


def test_preemption_gives_the_same_tokens(model_dirs):
    """With too few pages for all requests to finish together the youngest is preempted and
    recomputed; greedy tokens are those of an engine with plenty of pages."""
    from xinfer_amd import SamplingParams
    rng = random.Random(2)
    prompts = [harness.random_prompt(rng, n, 256) for n in (30, 31, 20)]
    sp = SamplingParams(temperature=0.0, max_tokens=40, ignore_eos=True)
    roomy = _engine(model_dirs["A"], "A", "f32", max_num_seqs=4, num_pages=40)
    want = [o.token_ids for o in roomy.generate(prompts, sp)]
    tight = _engine(model_dirs["A"], "A", "f32", max_num_seqs=4, num_pages=8)
    got = tight.generate(prompts, sp)
    assert [o.token_ids for o in got] == want
    assert tight.num_preemptions > 0 and roomy.num_preemptions == 0
    assert tight.get_available_kv_tokens() == 8 * 16
    # a request that could never fit, even alone, is refused when it is added
    small = _engine(model_dirs["A"], "A", "f32", max_num_seqs=2, num_pages=4)
    with pytest.raises(Exception, match="cache pages"):
        small.generate([harness.random_prompt(rng, 60, 256)], SamplingParams(max_tokens=30))


def test_running_ahead_gives_the_same_tokens(model_dirs):
    """The engine launches a step before it has read the tokens of the step before it (they reach the
    step on the device) and applies the finishing rules a step late; with `run_ahead=False` it
    reads every step's tokens first.  Both give the same tokens and reasons: greedy and sampled,
    with so few pages that requests are preempted and recomputed, with stop tokens and
    end-of-sequence ids (a request that ends has one token computed for nothing, which must not
    show), with length limits of 1 and 2 tokens, with penalties (whose steps wait for the tokens),
    and with requests cancelled while a step is on its way."""
    from xinfer_amd import SamplingParams
    rng = random.Random(3)
    prompts = [harness.random_prompt(rng, n, 509) for n in (1, 9, 64, 130, 200, 33, 77, 5)]
    stops = [[7], [100, 101], [3]] + [[t] for t in range(200, 260)]
    cases = [
        ("greedy", SamplingParams(temperature=0.0, max_tokens=24, ignore_eos=True), dict(num_pages=200)),
        ("sampled, few pages", SamplingParams(temperature=0.8, top_k=20, max_tokens=60, ignore_eos=True),
         dict(num_pages=36, max_num_seqs=6)),
        ("whole distribution", SamplingParams(temperature=1.1, top_p=0.9, max_tokens=20, ignore_eos=True), dict(num_pages=200)),
        ("stops", SamplingParams(temperature=0.9, max_tokens=60, ignore_eos=True, stop_token_ids=stops),
         dict(num_pages=200, max_num_seqs=8)),
        ("end of sequence", SamplingParams(temperature=0.9, max_tokens=60), dict(num_pages=200, eos=set(range(0, 509, 9)))),
        ("one token", SamplingParams(temperature=0.0, max_tokens=1, ignore_eos=True), dict(num_pages=200)),
        ("two tokens", SamplingParams(temperature=0.7, max_tokens=2, ignore_eos=True), dict(num_pages=200)),
        ("penalties", SamplingParams(temperature=0.7, max_tokens=30, ignore_eos=True, frequency_penalty=0.5), dict(num_pages=200)),
    ]
    for name, sp, kw in cases:
        kw = dict(kw)
        eos = kw.pop("eos", None)
        results = []
        for ahead in (False, True):
            eng = _engine(model_dirs["B"], "B", "f32", prefill_chunk_size=48, max_num_batched_tokens=64,
                          run_ahead=ahead, **{"max_num_seqs": 4, **kw})
            if eos is not None:
                eng.eos_token_ids = eos
            outs = eng.generate(prompts, sp)
            results.append(([(o.token_ids, o.finish_reason) for o in outs], eng.num_preemptions))
            assert eng.runner.cache.free_pages(0) == kw["num_pages"] and eng._launched is None, name
        assert results[0][0] == results[1][0], name
        if name == "sampled, few pages":
            assert results[0][1] > 0 and results[1][1] > 0
        if name in ("stops", "end of sequence"):
            reasons = {r for _, r in results[1][0]}
            assert ("stop" if name == "stops" else "eos") in reasons, reasons
    # cancelling while a step is on its way: the others go on as if nothing had happened
    sp = SamplingParams(temperature=0.0, max_tokens=20, ignore_eos=True)
    alone = _engine(model_dirs["B"], "B", "f32", max_num_seqs=4, num_pages=200).generate([prompts[2], prompts[5]], sp)
    eng = _engine(model_dirs["B"], "B", "f32", max_num_seqs=4, num_pages=200)
    rids = [eng.add_request(p, sp) for p in (prompts[2], prompts[3], prompts[5])]
    for _ in range(6):
        eng.step()
    assert eng._launched is not None
    eng.cancel(rids[1])
    eng.run_until_done()
    assert [eng._finished[r].generated for r in (rids[0], rids[2])] == [o.token_ids for o in alone]
    assert rids[1] not in eng._finished and eng.runner.cache.free_pages(0) == 200


def test_yarn_scaling_factor_stretches_the_positions(model_dirs):
    """`yarn_scaling_factor=2` (the reference's --yarn-scaling-factor) on the model of 128 positions:
    prompts of 150 and 200 tokens are taken, and the greedy tokens are those of the plain model under
    the rope_scaling that the option stands for (YaRN over 128 positions, beta_fast 32, beta_slow 1);
    without the option such a prompt is refused."""
    from xinfer_amd import SamplingParams
    rng = random.Random(6)
    prompts = [harness.random_prompt(rng, n, 256) for n in (150, 200, 9)]
    sp = SamplingParams(temperature=0.0, max_tokens=8, ignore_eos=True)
    with pytest.raises(ValueError, match="max_model_len"):
        _engine(model_dirs["A"], "A", "f32", max_num_seqs=4, num_pages=40).generate(prompts, sp)
    eng = _engine(model_dirs["A"], "A", "f32", max_num_seqs=4, num_pages=40, prefill_chunk_size=64, yarn_scaling_factor=2.0)
    assert eng.max_model_len == 256 and eng.model.spec.max_positions == 256
    outs = eng.generate(prompts, sp)
    pm = plain.PlainModel(model_dirs["A"])
    pm.config["rope_scaling"] = dict(rope_type="yarn", factor=2.0, original_max_position_embeddings=128,
                                     beta_fast=32.0, beta_slow=1.0, extrapolation_factor=1.0, attn_factor=1.0)
    for p, o in zip(prompts, outs):
        ids = list(p)
        for tok in o.token_ids:
            lg = pm.logits(ids)[-1]
            assert float(lg.max() - lg[tok]) < 1e-4
            ids.append(tok)
    plain_unscaled = plain.PlainModel(model_dirs["A"]).logits(prompts[2])
    assert not torch.allclose(pm.logits(prompts[2]), plain_unscaled, atol=1e-3)      # the scaling is at work from the start


def test_eos_and_limits(model_dirs):
    from xinfer_amd import SamplingParams
    eng = _engine(model_dirs["A"], "A", "f32", max_num_seqs=2, num_pages=16, max_model_len=40)
    prompt = [1, 2, 3, 4, 5]
    free_run = eng.generate([prompt], SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True))[0]
    assert free_run.decoded_length == 12
    eng.eos_token_ids = {free_run.token_ids[4]}
    cut = eng.generate([prompt], SamplingParams(temperature=0.0, max_tokens=12))[0]
    first = free_run.token_ids.index(free_run.token_ids[4])
    assert cut.token_ids == free_run.token_ids[:first] and cut.finish_reason == "eos"
    eng.eos_token_ids = set()
    long = eng.generate([prompt], SamplingParams(temperature=0.0, max_tokens=1000, ignore_eos=True))[0]
    assert long.prompt_length + long.decoded_length == 40          # clipped to max_model_len
    with pytest.raises(ValueError, match="max_model_len"):
        eng.generate([[1] * 40], SamplingParams(max_tokens=2))


def test_eos_ids_of_config_and_generation_config_both_stop(model_dirs, tmp_path):
    """config.json names one end-of-sequence id and generation_config.json a list with another:
    the engine stops on either (Config::apply_generation_cfg, /root/reference/src/utils/config.rs:360-375)."""
    import json
    import shutil
    from xinfer_amd import SamplingParams
    prompts = [[1, 2, 3, 4, 5], [9, 8, 7]]
    free = _engine(model_dirs["A"], "A", "f32", max_num_seqs=2, num_pages=16).generate(
        prompts, SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True))
    a, b = free[0].token_ids[5], free[1].token_ids[3]
    assert a not in free[1].token_ids[:4] and b not in free[0].token_ids[:6] and a != b
    d = tmp_path / "with_eos"
    shutil.copytree(model_dirs["A"], d)
    with open(d / "config.json") as f:
        raw = json.load(f)
    raw["eos_token_id"] = a
    (d / "config.json").write_text(json.dumps(raw))
    (d / "generation_config.json").write_text(json.dumps({"eos_token_id": [b, 255], "temperature": 0.6, "top_k": 20}))
    eng = _engine(str(d), "A", "f32", max_num_seqs=2, num_pages=16)
    assert eng.eos_token_ids == {a, b, 255}
    assert (eng.generation_cfg.temperature, eng.generation_cfg.top_k) == (0.6, 20)
    out = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=12))
    assert out[0].token_ids == free[0].token_ids[:free[0].token_ids.index(a)] and out[0].finish_reason == "eos"
    assert out[1].token_ids == free[1].token_ids[:free[1].token_ids.index(b)] and out[1].finish_reason == "eos"
    # one id instead of a list
    (d / "generation_config.json").write_text(json.dumps({"eos_token_id": b}))
    assert _engine(str(d), "A", "f32", max_num_seqs=2, num_pages=16).eos_token_ids == {a, b}


def test_engine_plans_pages_group_by_group(model_dirs):
    """Left to plan its cache itself, the engine gives tiny W's layers with a window of 24 pages for a
    window and a portion a request, its layer that keeps every key pages for the model's length,
    and generates the plain model's greedy tokens on that: with two long requests the window
    group's pages are used again and again."""
    from xinfer_amd import SamplingParams
    eng = _engine(model_dirs["W"], "W", "f32", max_num_seqs=2, max_model_len=320, prefill_chunk_size=32)
    assert [g.window for g in eng.model.cache_groups] == [24, 0]
    assert [g.num_pages for g in eng.runner.cache.groups] == [2 * (-(-(24 - 1 + 32) // 16) + 1), 2 * (320 // 16)]
    rng = random.Random(17)
    prompts = [harness.random_prompt(rng, n, 300) for n in (250, 301)]
    outs = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True))
    pm = plain.PlainModel(model_dirs["W"])
    for p, o in zip(prompts, outs):
        assert o.token_ids == pm.greedy(p, 12)
    assert eng.num_preemptions == 0 and eng.runner.cache.live_requests() == 0


# ---- streaming -----------------------------------------------------------------------------------
def test_streams_interleave_and_cancel(model_dirs):
    """Two streams read in turn give the tokens `generate` gives; a cancelled stream gives its
    pages back at once."""
    from xinfer_amd import Message, SamplingParams
    rng = random.Random(6)
    p1, p2 = harness.random_prompt(rng, 21, 256), harness.random_prompt(rng, 9, 256)
    sp = SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True)
    eng = _engine(model_dirs["A"], "A", "f32", max_num_seqs=3, num_pages=12, prefill_chunk_size=8)
    want = [o.token_ids for o in eng.generate([p1, p2], sp)]
    id1, n1, s1 = eng.generate_stream(sp, p1)
    id2, n2, s2 = eng.generate_stream(sp, p2)
    assert (n1, n2) == (21, 9) and id1 != id2 and s1.seq_id == id1
    got1, got2, done = [], [], []
    for a, b in zip(s1, s2):
        for item, got in ((a, got1), (b, got2)):
            if item.datatype == "TOKEN_ID":
                got.append(item.data)
            elif item.datatype == "DONE":
                done.append(item.data)
            else:
                assert item.datatype == "TOKEN" and isinstance(item.data, str)
    assert [got1, got2] == want and len(done) == 2 and done[0][3] == 10 and s1.finished and s2.finished
    _, _, s3 = eng.generate_stream(SamplingParams(temperature=0.0, max_tokens=50, ignore_eos=True),
                                   [Message("user", "hello there")])
    first = [next(s3) for _ in range(4)]
    assert [i.datatype for i in first] == ["TOKEN_ID", "TOKEN"] * 2
    assert eng.get_available_kv_tokens() < 12 * 16
    s3.cancel()
    assert s3.cancelled and list(s3) == []
    assert eng.get_available_kv_tokens() == 12 * 16 and eng.runner.cache.live_requests() == 0
    # a request that is not streamed: one COMPLETION item with its times and all its tokens
    _, _, s4 = eng.generate_stream(sp, p1, completion=True)
    items = list(s4)
    assert [i.datatype for i in items] == ["COMPLETION"] and items[0].data[3] == want[0] and len(items[0].data) == 4
    assert s4.finished and eng.runner.cache.live_requests() == 0


def test_stream_text_is_the_text_of_all_tokens(model_dirs, tmp_path):
    """With a byte-level tokenizer in the model folder the generated bytes are mostly halves of
    characters: text that is held back when the request ends comes as a last TOKEN item, so the
    pieces joined are what one decode of all tokens gives."""
    import shutil
    from tokenizers import Tokenizer, decoders, models, pre_tokenizers
    from xinfer_amd import SamplingParams
    d = tmp_path / "with_tokenizer"
    shutil.copytree(model_dirs["A"], d)
    vocab = {c: i for i, c in enumerate(sorted(pre_tokenizers.ByteLevel.alphabet()))}
    tok = Tokenizer(models.BPE(vocab=vocab, merges=[]))
    tok.pre_tokenizer = pre_tokenizers.ByteLevel(add_prefix_space=False)
    tok.decoder = decoders.ByteLevel()
    tok.save(str(d / "tokenizer.json"))
    eng = _engine(str(d), "A", "f32", max_num_seqs=2, num_pages=12)
    held = 0
    for seed in range(4):
        prompt = harness.random_prompt(random.Random(60 + seed), 12, 256)
        _, _, stream = eng.generate_stream(SamplingParams(temperature=1.0, max_tokens=9, ignore_eos=True, seed=seed), prompt)
        ids, pieces, kinds = [], [], []
        for item in stream:
            kinds.append(item.datatype)
            if item.datatype == "TOKEN_ID":
                ids.append(item.data)
            elif item.datatype == "TOKEN":
                pieces.append(item.data)
        assert kinds[-1] == "DONE" and len(ids) == 9
        assert "".join(pieces) == eng.tokenizer.decode(ids)
        held += len(pieces) > len(ids)
    assert held > 0         # some request did end inside a character


# ---- the command line ----------------------------------------------------------------------------
def test_command_line(model_dirs, capsys):
    """`python -m xinfer_amd` with the reference's option names: prompts as text (the folder has
    no tokenizer.json, so bytes are the tokens) and as token ids, greedy, and the two
    throughput lines of the reference's output."""
    from xinfer_amd import cli
    rc = cli.main(["--w", model_dirs["A"], "--prompts", "How are you?|Tell me", "--max-tokens", "6",
                   "--max-model-len", "64", "--temperature", "0", "--ignore-eos", "--page-size", "16",
                   "--num-pages", "8", "--dtype", "f32"])
    out = capsys.readouterr().out
    assert rc == 0
    assert "[Prompt 1]" in out and "[Prompt 2]" in out and "Response:" in out
    assert "Prompt tokens: 19 in" in out and "Decoded tokens: 12 in" in out
    rc = cli.main(["--m", model_dirs["A"], "--prompt-ids", "1,2,3|4,5", "--max-tokens", "4", "--max-model-len", "32",
                   "--seed", "3", "--page-size", "16", "--num-pages", "4", "--batch", "3", "--ignore-eos"])
    out = capsys.readouterr().out
    assert rc == 0 and "Decoded tokens: 12 in" in out and "[Prompt 1]" not in out     # --batch repeats the first prompt
    assert cli.main(["--m", model_dirs["A"], "--w", model_dirs["A"]]) == 2
    assert cli.main([]) == 2


def test_command_line_interactive_chat(model_dirs, monkeypatch, capsys):
    """`--i`: lines from the input are the user's turns of one conversation; the second answer
    has the first exchange in its context; the end of the input clears the history, a second
    end exits.  Greedy, so the first answer equals the one `generate_stream` gives for the
    same chat."""
    from xinfer_amd import Engine, EngineConfig, Message, SamplingParams, cli
    lines = iter(["Hello there", "", "And again"])

    def fake_input():
        try:
            return next(lines)
        except StopIteration:
            raise EOFError

    monkeypatch.setattr("builtins.input", fake_input)
    rc = cli.main(["--m", model_dirs["A"], "--i", "--max-tokens", "5", "--max-model-len", "128", "--temperature", "0",
                   "--ignore-eos", "--page-size", "16", "--num-pages", "16", "--dtype", "f32"])
    out = capsys.readouterr().out
    assert rc == 0
    assert out.count("Enter a new prompt") == 2 and out.count("Enter another prompt") == 3
    assert "No prompt was given." in out and "Chat history cleared" in out and out.rstrip().endswith("Exiting.")
    left = [int(l.split(":")[1]) for l in out.splitlines() if l.startswith("Tokens left:")]
    assert len(left) == 2 and left[1] < left[0] < 128
    engine = Engine(EngineConfig(model_id=model_dirs["A"], max_model_len=128, max_tokens=5, page_size=16, num_pages=16), "f32")
    _, _, stream = engine.generate_stream(SamplingParams(temperature=0.0, ignore_eos=True), [Message("user", "Hello there")])
    first = "".join(it.data for it in stream if it.datatype == "TOKEN")
    assert first in out


def test_stop_sequences(model_dirs):
    """Generation ends at the token that completes a stop sequence, which is not appended; the
    first tokens of a longer stop sequence stay; a stop that never completes changes nothing."""
    from xinfer_amd import Engine, EngineConfig, SamplingParams
    cfg = EngineConfig(model_id=model_dirs["A"], max_model_len=64, max_num_seqs=4, page_size=16, num_pages=16)
    engine = Engine(cfg, "f32")
    prompt = [5, 17, 3, 9]
    # sampled with a seed of the request's own: the same tokens in every run, and varied ones
    greedy = dict(temperature=1.5, seed=7, ignore_eos=True, max_tokens=12)
    full = engine.generate([prompt], SamplingParams(**greedy))[0].token_ids
    assert len(full) == 12
    k = next(i for i in range(2, 12) if full[i] not in full[:i])            # its first occurrence is at i
    one = engine.generate([prompt], SamplingParams(stop_token_ids=[[full[k]]], **greedy))[0]
    assert one.token_ids == full[:k] and one.finish_reason == "stop"
    j = next(i for i in range(2, 12) if full[i - 1:i + 1] not in [full[a - 1:a + 1] for a in range(1, i)])
    two = engine.generate([prompt], SamplingParams(stop_token_ids=[[full[j - 1], full[j]]], **greedy))[0]
    assert two.token_ids == full[:j] and two.finish_reason == "stop"
    never = engine.generate([prompt], SamplingParams(stop_token_ids=[[full[3], full[3] + 1 if full[4] != full[3] + 1 else full[3] + 2]],
                                                      **greedy))[0]
    assert never.token_ids == full and never.finish_reason == "length"
    # as text: the byte tokenizer maps a character below 128 to the token of its code
    low = [i for i in range(1, 12) if full[i] < 128 and full[i] not in full[:i] and chr(full[i]).isprintable()]
    if low:
        txt = engine.generate([prompt], SamplingParams(stop_sequences=["", chr(full[low[0]])], **greedy))[0]
        assert txt.token_ids == full[:low[0]] and txt.finish_reason == "stop"


# ---- long decoding and first tokens ----------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_one_by_one(dtype, model_dirs):
    """A whole sequence up to the model's last position fed one token per step, with a second
    request decoding beside it, against the plain logits."""
    from xinfer_amd.engine import ModelRunner, StepEntry, load_model
    name = "B"
    rng = random.Random(3)
    a = harness.random_prompt(rng, 512, 509)
    b = harness.random_prompt(rng, 300, 509)
    pm = plain.PlainModel(model_dirs[name])
    ref = {"a": pm.logits(a), "b": pm.logits(b)}
    runner = ModelRunner(load_model(model_dirs[name], dtype, DEV), page_size=8, num_pages=64 + 38, max_requests=2)
    runner.add_request(0)
    runner.add_request(1)
    got = {}
    for i in range(512):
        entries = [StepEntry(0, [a[i]], [0])]
        if i < 300:
            entries.append(StepEntry(1, [b[i]], [0]))
        lg = runner.step(entries).cpu()
        got[("a", i)] = lg[0]
        if i < 300:
            got[("b", i)] = lg[1]
    harness.compare(got, ref, harness.TOL[dtype], f"long decoding {dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(TINY))
def test_first_tokens(name, dtype, model_dirs):
    """The first positions of a sequence (one key, two keys, ...) alone in a step."""
    from xinfer_amd.engine import ModelRunner, StepEntry, load_model
    vocab = TINY[name]["config"]["vocab_size"]
    toks = [vocab - 1, 0, 7, 7]
    pm = plain.PlainModel(model_dirs[name])
    ref = {"x": pm.logits(toks)}
    runner = ModelRunner(load_model(model_dirs[name], dtype, DEV), TINY[name]["page_size"], 2, 1)
    runner.add_request(0)
    got = {("x", i): runner.step([StepEntry(0, [t], [0])]).cpu()[0] for i, t in enumerate(toks)}
    harness.compare(got, ref, harness.TOL[dtype], f"first tokens {name} {dtype}")


def test_bfloat16_cache_keeps_values_in_groups_of_eight_keys(model_dirs):
    """The bfloat16 path keeps V as [pages, kv heads, page / 8, head_dim, 8] (what its matrix-core kernels read), the
    32-bit path as [pages, kv heads, page, head_dim]; a page that is no multiple of 8 tokens is refused in bfloat16 with a
    clear error and runs in 32 bits."""
    from xinfer_amd.engine import ModelRunner, StepEntry, load_model
    cfg = TINY["A"]["config"]
    nkv, d = cfg["num_key_value_heads"], cfg["head_dim"]
    model = load_model(model_dirs["A"], "bfloat16", DEV)
    runner = ModelRunner(model, page_size=16, num_pages=3, max_requests=1)
    lc = next(iter(runner.layer_caches.values()))
    assert tuple(lc.k.shape) == (3, nkv, 16, d) and tuple(lc.v.shape) == (3, nkv, 2, d, 8)
    with pytest.raises(ValueError, match="multiple of 8"):
        ModelRunner(model, page_size=12, num_pages=3, max_requests=1)
    wide = ModelRunner(load_model(model_dirs["A"], "float32", DEV), page_size=12, num_pages=3, max_requests=1)
    lc = next(iter(wide.layer_caches.values()))
    assert tuple(lc.v.shape) == tuple(lc.k.shape) == (3, nkv, 12, d)
    wide.add_request(0)
    assert torch.isfinite(wide.step([StepEntry(0, list(range(1, 20)), [18])])).all()


def test_step_refuses_bad_input(model_dirs):
    from xinfer_amd.cache import OutOfPages
    from xinfer_amd.engine import ModelRunner, StepEntry, StepError, load_model
    runner = ModelRunner(load_model(model_dirs["A"], "float32", DEV), 16, 2, 2)
    runner.add_request(0)
    for entries, needle in [([StepEntry(0, [], [])], "at least one"), ([StepEntry(0, [256], [0])], "vocabulary"),
                            ([StepEntry(0, [1], [1])], "outside"), ([StepEntry(3, [1], [0])], "not live"),
                            ([StepEntry(0, [1], []), StepEntry(0, [2], [])], "twice"),
                            ([StepEntry(0, [1] * 129, [])], "positions")]:
        with pytest.raises(StepError, match=needle):
            runner.step(entries)
    with pytest.raises(OutOfPages):
        runner.step([StepEntry(0, [1] * 40, [])])
    assert runner.length(0) == 0 and runner.cache.free_pages(0) == 2
    runner.cache.check()


# ---- decode steps recorded as HIP graphs ---------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,n_req", [("B", 3), ("W", 12)])
def test_decode_graph_replays_equal_launch_by_launch(name, n_req, dtype, model_dirs):
    """Decode steps replayed from a recorded graph give, bit for bit, the logits of the same
    steps launched kernel by kernel: over many replays, with prompt portions of other requests
    run between them (the program's own launch-by-launch work), with requests that end and
    join (so the batch size, and with it the graph, changes), and with pages used again.
    Twelve requests make the matrix products go through the vendor library inside the graph."""
    from xinfer_amd.engine import ModelRunner, StepEntry, load_model
    t = TINY[name]
    vocab, page = t["config"]["vocab_size"], t["page_size"]
    model = load_model(model_dirs[name], dtype, DEV)
    rng = random.Random(77)
    prompts = {i: harness.random_prompt(rng, rng.randrange(3, 60), vocab) for i in range(n_req + 2)}
    feed = {i: harness.random_prompt(rng, 40, vocab) for i in prompts}

    def run(use_graphs):
        runner = ModelRunner(model, page, 16 * (n_req + 2), n_req + 2, use_graphs=use_graphs, graph_after=1)
        out = []
        live = list(range(n_req))
        for i in live:
            runner.add_request(i)
            runner.step([StepEntry(i, prompts[i], [])])
        for step in range(36):
            if step == 9:                            # one ends; its pages go back
                runner.release(live.pop(1))
            if step == 14:                           # another joins: a prompt portion between replays
                j = n_req
                runner.add_request(j)
                out.append(runner.step([StepEntry(j, prompts[j][:2], [1])]).cpu())
                out.append(runner.step([StepEntry(j, prompts[j][2:], [0])]).cpu())
                live.append(j)
            entries = [StepEntry(i, [feed[i][step]], [0] if (i + step) % 5 else []) for i in live]
            out.append(runner.step(entries).cpu())
        runner.cache.check()
        return out, runner

    want, r0 = run(False)
    got, r1 = run(True)
    # a step that records a graph runs launch by launch; every later step of its kind is a replay
    assert r0.graph_replays == 0 and r1.graphs_dropped == 0 and r1.graph_replays == 36 - len(r1._graphs)
    assert len(want) == len(got)
    for k, (a, b) in enumerate(zip(want, got)):
        assert a.shape == b.shape and torch.equal(a, b), f"step {k} differs between graph and launches"


def test_a_batch_size_is_recorded_the_third_time_it_is_seen(model_dirs):
    from xinfer_amd.engine import ModelRunner, StepEntry, load_model
    runner = ModelRunner(load_model(model_dirs["A"], "bfloat16", DEV), 16, 8, 2)
    runner.add_request(0)
    runner.add_request(1)
    for step in range(5):
        runner.step([StepEntry(0, [step], [0]), StepEntry(1, [step + 7], [0])])
        assert (len(runner._graphs), runner.graph_replays) == ((0, 0) if step < 2 else (1, step - 2))
    runner.release(1)
    runner.step([StepEntry(0, [9], [0])])                      # another batch size: first sighting
    assert (len(runner._graphs), runner.graph_replays) == (1, 2)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_graphs_across_a_bucket_edge(dtype, tmp_path):
    """A request grows from 1,021 to 1,030 keys: the steps up to 1,024 replay the graph of the
    1,024 bucket, the later ones that of 2,048 (whose attention grid is laid out for 2,048 keys).
    Every replayed step against the same step launched kernel by kernel, bit for bit, stopping at
    the first difference, and against the plain model."""
    from xinfer_amd.engine import ModelRunner, StepEntry, load_model
    from xinfer_amd.weights import write_random_model
    t = TINY["B"]
    cfg = dict(t["config"], max_position_embeddings=2048)
    d = write_random_model(str(tmp_path / "b2048"), cfg, t["seed"], t["linear_std"], t["norm_std"])
    vocab, page = cfg["vocab_size"], t["page_size"]
    model = load_model(d, dtype, DEV)
    rng = random.Random(5)
    long = harness.random_prompt(rng, 1030, vocab)
    short = harness.random_prompt(rng, 40, vocab)

    def run(use_graphs):
        runner = ModelRunner(model, page, 2048 // page + 8, 2, use_graphs=use_graphs, graph_after=1)
        runner.add_request(0)
        runner.add_request(1)
        runner.step([StepEntry(0, long[:1020], []), StepEntry(1, short[:30], [])])
        out = [runner.step([StepEntry(0, [long[1020 + k]], [0]), StepEntry(1, [short[30 + k]], [0])]).cpu() for k in range(10)]
        return out, runner

    want, _ = run(False)
    got, runner = run(True)
    assert sorted(runner._graphs) == [(2, 1024, False), (2, 2048, False)] and runner.graph_replays == 8
    for k, (a, b) in enumerate(zip(want, got)):
        assert torch.equal(a, b), f"the step that makes {1021 + k} keys differs between graph and launches"
    ref = plain.PlainModel(d).logits(long)
    scale = float(ref.abs().max())
    for k, a in enumerate(got):
        assert float((a[0] - ref[1020 + k]).abs().max()) < harness.TOL[dtype] * scale, 1021 + k


def test_recorded_graphs_are_bounded(model_dirs):
    """With room for two graphs the least recently used one goes when a third is recorded; its
    batch size is recorded again when it comes back, and the logits stay those of launched steps."""
    from xinfer_amd.engine import ModelRunner, StepEntry, load_model
    model = load_model(model_dirs["A"], "bfloat16", DEV)

    def run(**kw):
        runner = ModelRunner(model, 16, 12, 3, graph_after=1, **kw)
        out = []
        for i in range(3):
            runner.add_request(i)
        for step, live in enumerate([[0], [0], [0, 1], [0], [0, 1, 2], [0, 1, 2], [0, 1], [0, 1]]):
            out.append(runner.step([StepEntry(i, [step + 3 * i], [0]) for i in live]).cpu())
        return out, runner

    want, _ = run(use_graphs=False)
    got, runner = run(graphs_most=2)
    assert all(torch.equal(a, b) for a, b in zip(want, got))
    # sizes 1, 2 recorded; 1 used again; 3 recorded: 2 goes; 2 recorded again: 1 goes
    assert [k[0] for k in runner._graphs] == [3, 2] and runner.graphs_dropped == 2 and runner.graph_replays == 4
    got, runner = run(graph_bytes_most=1)          # no room beyond the graph in use
    assert all(torch.equal(a, b) for a, b in zip(want, got))
    assert len(runner._graphs) == 1 and runner.graphs_dropped == 4


def test_sizes_the_decode_kernel_does_not_take_are_not_recorded(tmp_path):
    """32 query heads on one kv head: the split-K decode kernel takes up to 16 per kv head, so the
    prefill kernel serves single tokens too, and it reads the step's lengths on the host: the model
    says so and its steps are launched one by one, many times over."""
    from xinfer_amd.engine import ModelRunner, StepEntry, load_model
    from xinfer_amd.weights import write_random_model
    cfg = dict(TINY["B"]["config"], num_attention_heads=32, num_key_value_heads=1, head_dim=16, hidden_size=64,
               num_hidden_layers=1)
    d = write_random_model(str(tmp_path / "g32"), cfg, 3, 0.05, 0.1)
    model = load_model(d, "bfloat16", DEV)
    assert not model.graph_safe and load_model(d, "float32", DEV).graph_safe
    runner = ModelRunner(model, 8, 16, 2, graph_after=2)
    assert not runner.use_graphs
    toks = harness.random_prompt(random.Random(1), 30, cfg["vocab_size"])
    runner.add_request(0)
    got = [runner.step([StepEntry(0, toks[:20], [19])]).cpu()[0]]
    got += [runner.step([StepEntry(0, [toks[20 + k]], [0])]).cpu()[0] for k in range(10)]
    ref = plain.PlainModel(d).logits(toks)
    for k, a in enumerate(got):
        assert float((a - ref[19 + k]).abs().max()) < harness.TOL["bfloat16"] * float(ref.abs().max())
    assert runner.graph_replays == 0


def test_model_with_a_part_that_reads_the_host_is_not_recorded(model_dirs):
    from xinfer_amd.engine import ModelRunner, load_model
    model = load_model(model_dirs["A"], "bfloat16", DEV)
    assert model.graph_safe and ModelRunner(model, 16, 4, 2).use_graphs
    model.blocks[0].mixer.graph_safe = False
    assert not model.graph_safe and not ModelRunner(model, 16, 4, 2).use_graphs


# ---- the replay program ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(dtype, model_dirs, tmp_path):
    """bin/trace_run as a user runs it: steps on standard input, `done <step>` lines back,
    <step>.f32 files with [wanted, vocab] little-endian float32."""
    name = "A"
    reqs = {f"r{i}": harness.random_prompt(random.Random(40 + i), n, 256) for i, n in enumerate([33, 70, 5, 64, 100])}
    steps = harness.trace_mixed(reqs, 3)
    need = harness.tokens_needed(steps, 64)
    out = tmp_path / "out"
    proc = subprocess.Popen(
        [sys.executable, os.path.join(REPO, "bin", "trace_run"), "--model", model_dirs[name], "--dtype", dtype,
         "--out", str(out), "--max-tokens", str(need)],
        stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    for st in steps:
        proc.stdin.write(json.dumps(st) + "\n")
        proc.stdin.flush()
        assert proc.stdout.readline().strip() == f"done {st['step']}"
    proc.stdin.close()
    assert proc.wait(timeout=120) == 0
    pm = plain.PlainModel(model_dirs[name])
    ref = {rid: pm.logits(t) for rid, t in reqs.items()}
    got, fed = {}, {rid: 0 for rid in reqs}
    for st in steps:
        wanted = sum(len(e["want"]) for e in st["entries"])
        arr = np.fromfile(out / f"{st['step']}.f32", dtype="<f4").reshape(wanted, 256)
        row = 0
        for e in st["entries"]:
            for w in e["want"]:
                got[(e["id"], fed[e["id"]] + w)] = torch.from_numpy(arr[row].copy())
                row += 1
            fed[e["id"]] += len(e["tokens"])
    assert len(got) == sum(len(t) for t in reqs.values())
    harness.compare(got, ref, harness.TOL[dtype], f"trace_run {dtype}")


# ---- parts alone ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_parts_alone(dtype, model_dirs):
    """Norm, feed-forward and attention mixer of tiny W's layer 0 each against its plain function."""
    from xinfer_amd.engine import ModelRunner, StepEntry, load_model
    name = "W"
    model = load_model(model_dirs[name], dtype, DEV)
    pm = plain.PlainModel(model_dirs[name])
    c, W = pm.config, pm.weights
    blk = model.blocks[0]
    g = torch.Generator().manual_seed(12)
    T, H = 37, c["hidden_size"]
    tol = 2e-5 if dtype == torch.float32 else 2.0 ** -7
    x = torch.randn(T, H, generator=g)
    # norm
    out = blk.norm1.forward(x.to(DEV).clone(), None, dtype).cpu().float()
    ref = plain.rms_norm(x, W["model.layers.0.input_layernorm.weight"], c["rms_norm_eps"])
    assert float((out - ref).abs().max() / ref.abs().max()) < tol
    # feed-forward
    xin = x.to(dtype)
    def whole(y):      # a part may answer with a stack of float32 partial sums for the next norm to add
        return (y.sum(0) if y.dim() == 3 else y).cpu().float()
    out = whole(blk.ffn.forward(xin.to(DEV), None))
    ref = plain.mlp_block(xin.float(), W, "model.layers.0.mlp")
    assert float((out - ref).abs().max() / ref.abs().max()) < 2 * tol
    # attention mixer with a window of 24 over 37 tokens, through the runner's own cache plumbing
    runner = ModelRunner(model, 16, 4, 1)
    runner.add_request(0)
    runner.cache.reserve(0, T)
    ctx = runner._context(runner.cache.build_batch([0], [T]), np.zeros(T, np.int32), np.zeros(0, np.int32))[0]
    out = whole(blk.mixer.forward(xin.to(DEV), ctx, runner.layer_caches[0]))
    cos, sin = plain.rope_tables(float(c["rope_theta"]), c["head_dim"], c["max_position_embeddings"])
    ref = plain.attention_block(xin.float(), W, "model.layers.0.self_attn", c, torch.arange(T), cos, sin, 24)
    assert float((out - ref).abs().max() / ref.abs().max()) < 2 * tol


# ---- a toy mixer with state of its own, registered from here ----------------------------------------------
def test_toy_mixer_with_state_registers_builds_and_steps(tmp_path):
    """A mixer defined in this test keeps a running sum of its inputs per request in a
    fixed-size state slot (no pages).  A new architecture using it in one layer, beside a
    normal attention layer, is registered, written as a random model folder, loaded and
    stepped in portions and mixed batches, without a change to the framework's files."""
    from dataclasses import dataclass
    from xinfer_amd.config.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry
    from xinfer_amd.engine import ModelRunner, StepEntry, load_model
    from xinfer_amd.models import ModelFamily, register_architecture
    from xinfer_amd.parts import Mixer, StateNeed, register_mixer
    from xinfer_amd.weights import TensorDecl, write_random_model

    @register_mixer("running_mean")
    class RunningMean(Mixer):
        """y[t] = W @ mean(x[0..t]) of the request: the state is (sum, count)."""

        def __init__(self, spec, dtype):
            super().__init__(spec, dtype)
            self.h = int(spec["hidden_size"])

        @classmethod
        def declare(cls, spec, prefix):
            return [TensorDecl(f"{prefix}.mix.weight", (int(spec["hidden_size"]),) * 2)]

        def load(self, store, prefix, device):
            self.w = store.get(f"{prefix}.mix.weight", torch.float32, device)

        def state_need(self):
            return StateNeed((self.h + 1,), torch.float32)

        def forward(self, x, ctx, cache):
            out = torch.empty((ctx.num_tokens, self.h), dtype=torch.float32, device=x.device)
            for b in range(ctx.num_seqs):
                lo, hi = ctx.cu_q_host[b], ctx.cu_q_host[b + 1]
                slot = int(ctx.state_slots[b])
                first_pos = ctx.ctx_lens_host[b] - (hi - lo)
                if first_pos == 0:
                    cache.state[slot].zero_()                       # a slot used before starts clean
                st = cache.state[slot]
                sums = st[:self.h] + torch.cumsum(x[lo:hi].float(), 0)
                counts = st[self.h] + torch.arange(1, hi - lo + 1, device=x.device)
                out[lo:hi] = (sums / counts[:, None]) @ self.w.T
                st[:self.h] = sums[-1]
                st[self.h] = counts[-1]
            return out.to(self.dtype)

    @dataclass(frozen=True)
    class ToyConfig:
        vocab_size: int
        hidden_size: int
        architecture: str = "ToyStateForCausalLM"

        @classmethod
        def from_dict(cls, raw, where="config.json"):
            return cls(int(raw["vocab_size"]), int(raw["hidden_size"]))

        def to_dict(self):
            return {"architectures": [self.architecture], "vocab_size": self.vocab_size,
                    "hidden_size": self.hidden_size}

    def toy_spec(cfg):
        h = cfg.hidden_size
        norm = PartSpec("rmsnorm", dict(dim=h, eps=1e-5))
        ffn = PartSpec("gated_mlp", dict(hidden_size=h, intermediate_size=2 * h, activation="silu"))
        rope = PartSpec("rope", dict(head_dim=16, rotary_dim=16, theta=10000.0, max_positions=256))
        attn = PartSpec("attention", dict(hidden_size=h, num_heads=2, num_kv_heads=1, head_dim=16, qk_norm=False,
                                          window=None, position=rope, scale=0.25))
        layers = (
            LayerSpec("model.layers.0", "prenorm", PartSpec("running_mean", dict(hidden_size=h)), ffn,
                      {"input_layernorm": norm, "post_attention_layernorm": norm}),
            LayerSpec("model.layers.1", "prenorm", attn, ffn,
                      {"input_layernorm": norm, "post_attention_layernorm": norm}))
        return ModelSpec(
            architecture=cfg.architecture, vocab_size=cfg.vocab_size, hidden_size=h, max_positions=256,
            embedding=PartSpec("embedding", dict(name="model.embed_tokens.weight", vocab_size=cfg.vocab_size, dim=h)),
            # layer 1 runs twice; its second run reads the keys and values its first run stored
            layers=layers, schedule=(ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(1, cache_of=1)),
            final_norm=PartSpec("rmsnorm", dict(dim=h, eps=1e-5, name="model.norm.weight")),
            head=PartSpec("lm_head", dict(name="lm_head.weight", tied=False, vocab_size=cfg.vocab_size, dim=h)))

    register_architecture("ToyStateForCausalLM", ModelFamily("toy", ToyConfig, toy_spec))
    d = write_random_model(str(tmp_path / "toy"), {"architectures": ["ToyStateForCausalLM"], "vocab_size": 97,
                                                   "hidden_size": 32}, seed=3, linear_std=0.1)
    model = load_model(d, "float32", DEV)
    assert set(model.state_needs) == {0} and set(model.kv_needs) == {1}

    def run(steps):
        runner = ModelRunner(model, page_size=8, num_pages=12, max_requests=2)
        return harness.replay(runner, steps)

    # the same model written out plainly, whole sequences
    W = plain.read_weights(d)
    cos, sin = plain.rope_tables(10000.0, 16, 256)

    def mlp(x, i):
        return plain.mlp_block(x, W, f"model.layers.{i}.mlp")

    def toy_logits(ids):
        T = len(ids)
        x = W["model.embed_tokens.weight"][torch.tensor(ids)]
        h = plain.rms_norm(x, W["model.layers.0.input_layernorm.weight"], 1e-5)
        mean = torch.cumsum(h, 0) / torch.arange(1, T + 1)[:, None]
        r = x + mean @ W["model.layers.0.self_attn.mix.weight"].T
        x = r + mlp(plain.rms_norm(r, W["model.layers.0.post_attention_layernorm.weight"], 1e-5), 0)
        kv = None
        for _ in range(2):
            h = plain.rms_norm(x, W["model.layers.1.input_layernorm.weight"], 1e-5)
            pos = torch.arange(T)
            q = plain.apply_rope((h @ W["model.layers.1.self_attn.q_proj.weight"].T).reshape(T, 2, 16), pos, cos, sin)
            if kv is None:
                k = plain.apply_rope((h @ W["model.layers.1.self_attn.k_proj.weight"].T).reshape(T, 1, 16), pos, cos, sin)
                kv = (k, (h @ W["model.layers.1.self_attn.v_proj.weight"].T).reshape(T, 1, 16))
            a = plain.attention(q, kv[0], kv[1], scale=0.25).reshape(T, 32)
            r = x + a @ W["model.layers.1.self_attn.o_proj.weight"].T
            x = r + mlp(plain.rms_norm(r, W["model.layers.1.post_attention_layernorm.weight"], 1e-5), 1)
        return plain.rms_norm(x, W["model.norm.weight"], 1e-5) @ W["lm_head.weight"].T

    rng = random.Random(9)
    reqs = {f"q{i}": harness.random_prompt(rng, n, 97) for i, n in enumerate([19, 40, 7, 33])}
    ref = {rid: toy_logits(t) for rid, t in reqs.items()}
    for what, steps in (("whole", harness.trace_whole(reqs)), ("mixed", harness.trace_mixed(reqs, 1, max_live=2)),
                        ("portions", harness.trace_portions(reqs))):
        harness.compare(run(steps), ref, harness.TOL["float32"], f"toy {what}")


# ---- a toy mixer with one paged pool of its own, a scaled embedding, a head kind registered from here ----------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_one_pool_cache_scaled_embedding_and_a_head_kind(dtype, tmp_path):
    """Data alone, beside part kinds registered here: (1) a mixer that keeps one pool of latent rows
    (no keys and values: `KVNeed(window, (PoolNeed("latent", (PAGE, L), float32),))`) and answers
    with the mean of the last `window` latents, read from the pages through the block table; (2)
    the built-in embedding with a `scale`; (3) a head kind of its own (a bias, then the built-in soft
    cap), registered from here; (4) tensor names of the layer's parts that are not the usual ones.
    With an attention layer beside it the model has two cache groups of different pools.  Stepped
    in every way of cutting with few pages, and generated from through the scheduler, whose window
    group holds a window and a portion, not the whole request."""
    from dataclasses import dataclass
    from xinfer_amd import Engine, EngineConfig, SamplingParams, kernels
    from xinfer_amd.config.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry
    from xinfer_amd.engine import ModelRunner, load_model
    from xinfer_amd.models import ModelFamily, register_architecture
    from xinfer_amd.parts import PAGE, KVNeed, Mixer, PoolNeed, register_head, register_mixer
    from xinfer_amd.parts.embedding import LMHead
    from xinfer_amd.weights import TensorDecl, write_random_model

    H, L, WINDOW, V, SCALE, CAP = 48, 12, 11, 131, 7.0, 3.0

    @register_mixer("latent_mean")
    class LatentMean(Mixer):
        def __init__(self, spec, dtype):
            super().__init__(spec, dtype)
            self.h, self.l, self.window = int(spec["hidden_size"]), int(spec["latent"]), int(spec["window"])

        @classmethod
        def declare(cls, spec, prefix):
            h, l = int(spec["hidden_size"]), int(spec["latent"])
            return [TensorDecl(f"{prefix}.down.weight", (l, h)), TensorDecl(f"{prefix}.up.weight", (h, l))]

        def load(self, store, prefix, device):
            self.down = store.get(f"{prefix}.down.weight", torch.float32, device)
            self.up = store.get(f"{prefix}.up.weight", torch.float32, device)

        def cache_need(self):
            return KVNeed(self.window, (PoolNeed("latent", (PAGE, self.l), torch.float32),))

        def forward(self, x, ctx, cache):
            pool = cache.pools["latent"]                                    # [pages, page_size, L]
            page = pool.shape[1]
            z = kernels.gemm_tn(x.float().contiguous(), self.down)
            pool.view(-1, self.l)[ctx.slots[cache.group]] = z               # this step's rows into their pages
            out = torch.empty((ctx.num_tokens, self.l), dtype=torch.float32, device=x.device)
            table = ctx.block_tables[cache.group]
            for b in range(ctx.num_seqs):
                lo, hi, n = ctx.cu_q_host[b], ctx.cu_q_host[b + 1], ctx.ctx_lens_host[b]
                for t in range(lo, hi):
                    p = n - (hi - t)                                         # the token's position
                    first = max(0, p - self.window + 1)
                    pos = torch.arange(first, p + 1, device=x.device)
                    rows = table[b][pos // page].long() * page + pos % page    # pages behind the window are gone (-1)
                    assert int(rows.min()) >= 0
                    out[t] = pool.view(-1, self.l)[rows].mean(0)
            return kernels.gemm_tn(out, self.up).to(self.dtype)

    @register_head("biased_head")
    class BiasedHead(LMHead):
        @classmethod
        def declare(cls, spec, prefix=""):
            return LMHead.declare(spec) + [TensorDecl(spec["bias_name"], (int(spec["vocab_size"]),))]

        def load(self, store, prefix, device, shared=None):
            super().load(store, prefix, device, shared=shared)
            self.bias = store.get(self.spec["bias_name"], torch.float32, device)

        def forward(self, h):
            logits = self.proj(h, out_dtype=torch.float32, skinny_rows=kernels.SKINNY_MAX_ROWS) + self.bias
            return kernels.softcap_(logits, self.softcap)

    @dataclass(frozen=True)
    class LatentConfig:
        vocab_size: int
        architecture: str = "ToyLatentForCausalLM"

        @classmethod
        def from_dict(cls, raw, where="config.json"):
            return cls(int(raw["vocab_size"]))

        def to_dict(self):
            return {"architectures": [self.architecture], "vocab_size": self.vocab_size}

    def latent_spec(cfg):
        norm = PartSpec("rmsnorm", dict(dim=H, eps=1e-5))
        ffn = PartSpec("gated_mlp", dict(hidden_size=H, intermediate_size=64, activation="silu"))
        rope = PartSpec("rope", dict(head_dim=16, rotary_dim=16, theta=10000.0, max_positions=256))
        attn = PartSpec("attention", dict(hidden_size=H, num_heads=3, num_kv_heads=1, head_dim=16, qk_norm=False,
                                          window=None, position=rope, scale=0.25))
        layers = (LayerSpec("blocks.0", "prenorm", PartSpec("latent_mean", dict(hidden_size=H, latent=L, window=WINDOW)), ffn,
                            {"ln_a": norm, "ln_b": norm}, mixer_name="mean", feed_forward_name="ff"),
                  LayerSpec("blocks.1", "prenorm", attn, ffn, {"ln_a": norm, "ln_b": norm}, mixer_name="attn",
                            feed_forward_name="ff"))
        return ModelSpec(
            architecture=cfg.architecture, vocab_size=cfg.vocab_size, hidden_size=H, max_positions=256,
            embedding=PartSpec("embedding", dict(name="wte.weight", vocab_size=cfg.vocab_size, dim=H, scale=SCALE)),
            layers=layers, schedule=(ScheduleEntry(0), ScheduleEntry(1)),
            final_norm=PartSpec("rmsnorm", dict(dim=H, eps=1e-5, name="ln_f.weight")),
            head=PartSpec("biased_head", dict(name="wte.weight", tied=True, vocab_size=cfg.vocab_size, dim=H,
                                              bias_name="head.bias", softcap=CAP)))

    register_architecture("ToyLatentForCausalLM", ModelFamily("toy_latent", LatentConfig, latent_spec))
    d = write_random_model(str(tmp_path / "latent"), {"architectures": ["ToyLatentForCausalLM"], "vocab_size": V},
                           seed=4, linear_std=0.15)
    model = load_model(d, dtype, DEV)
    assert [g.window for g in model.cache_groups] == [WINDOW, 0]
    assert [p.name for p in model.kv_needs[0].pools] == ["latent"] and [p.name for p in model.kv_needs[1].pools] == ["k", "v"]

    W = plain.read_weights(d)
    assert set(W) >= {"wte.weight", "head.bias", "blocks.0.mean.down.weight", "blocks.0.ln_a.weight", "blocks.1.attn.q_proj.weight",
                      "blocks.1.ff.down_proj.weight", "ln_f.weight"} and "lm_head.weight" not in W
    cos, sin = plain.rope_tables(10000.0, 16, 256)

    def toy_logits(ids):
        T = len(ids)
        x = W["wte.weight"][torch.tensor(ids)] * SCALE
        z = plain.rms_norm(x, W["blocks.0.ln_a.weight"], 1e-5) @ W["blocks.0.mean.down.weight"].T
        m = torch.stack([z[max(0, t - WINDOW + 1):t + 1].mean(0) for t in range(T)])
        r = x + m @ W["blocks.0.mean.up.weight"].T
        x = r + plain.mlp_block(plain.rms_norm(r, W["blocks.0.ln_b.weight"], 1e-5), W, "blocks.0.ff")
        h = plain.rms_norm(x, W["blocks.1.ln_a.weight"], 1e-5)
        pos = torch.arange(T)
        q = plain.apply_rope((h @ W["blocks.1.attn.q_proj.weight"].T).reshape(T, 3, 16), pos, cos, sin)
        k = plain.apply_rope((h @ W["blocks.1.attn.k_proj.weight"].T).reshape(T, 1, 16), pos, cos, sin)
        v = (h @ W["blocks.1.attn.v_proj.weight"].T).reshape(T, 1, 16)
        r = x + plain.attention(q, k, v, scale=0.25).reshape(T, 48) @ W["blocks.1.attn.o_proj.weight"].T
        x = r + plain.mlp_block(plain.rms_norm(r, W["blocks.1.ln_b.weight"], 1e-5), W, "blocks.1.ff")
        logits = plain.rms_norm(x, W["ln_f.weight"], 1e-5) @ W["wte.weight"].T + W["head.bias"]
        return CAP * torch.tanh(logits / CAP)

    rng = random.Random(19)
    reqs = {f"q{i}": harness.random_prompt(rng, n, V) for i, n in enumerate([21, 60, 5, 37, 90])}
    ref = {rid: toy_logits(t) for rid, t in reqs.items()}
    assert float(max(r.abs().max() for r in ref.values())) > 0.8 * CAP            # the cap is at work
    for what, steps in (("whole", harness.trace_whole(reqs)), ("mixed", harness.trace_mixed(reqs, 2, max_live=3)),
                        ("portions", harness.trace_portions(reqs)), ("tail", harness.trace_tail_one_by_one(reqs, tail=20))):
        need = harness.tokens_needed(steps, 8) // 8
        runner = ModelRunner(model, page_size=8, num_pages=[need, need], max_requests=3)
        got = harness.replay(runner, steps)
        assert runner.cache.free_pages(0) == need and runner.cache.free_pages(1) == need
        harness.compare(got, ref, harness.TOL[dtype], f"toy latent {dtype} {what}")

    # through the scheduler: the window group's pool holds a window and a portion (11 - 1 + 16 tokens: 4 pages and
    # one more), far less than the requests' lengths; greedy tokens are the plain model's
    if dtype == "float32":
        eng = Engine(EngineConfig(weight_path=d, page_size=8, num_pages=[2 * 5 + 1, 40], max_num_seqs=2, prefill_chunk_size=16,
                                  max_num_batched_tokens=24), dtype)
        prompts = [reqs["q1"], reqs["q4"][:70]]
        outs = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True))
        for p, o in zip(prompts, outs):
            ids = list(p)
            for tok in o.token_ids:
                lg = toy_logits(ids)[-1]
                assert float(lg.max() - lg[tok]) < 1e-4
                ids.append(tok)
        assert eng.runner.cache.free_pages(0) == 11 and eng.runner.cache.free_pages(1) == 40


# ---- a toy feed-forward with routing and a toy position encoding, registered from here --------------------
def test_toy_routed_feed_forward_and_position_encoding(tmp_path):
    """Two more part kinds defined in this test: a feed-forward that routes every token to the
    one of three gated experts whose router logit (float32) is largest, and a position encoding
    that rotates interleaved pairs of a part of the head by the position divided by a factor.  An
    architecture that uses them beside the built-in parts (the routed feed-forward in one layer,
    a dense one in the other) is registered, written, loaded and stepped in every way of cutting,
    without a change to the framework's files."""
    from dataclasses import dataclass
    from xinfer_amd.config.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry
    from xinfer_amd.engine import ModelRunner, load_model
    from xinfer_amd.models import ModelFamily, register_architecture
    from xinfer_amd.parts import FeedForward, PositionEncoding, register_feed_forward, register_position_encoding
    from xinfer_amd.weights import TensorDecl, write_random_model
    from xinfer_amd import kernels

    E, H, I, D, ROT, FACTOR, THETA = 3, 40, 24, 16, 8, 4.0, 500.0

    @register_feed_forward("top1_experts")
    class Top1Experts(FeedForward):
        def __init__(self, spec, dtype):
            super().__init__(spec, dtype)
            self.h, self.i, self.e = int(spec["hidden_size"]), int(spec["intermediate_size"]), int(spec["experts"])

        @classmethod
        def declare(cls, spec, prefix):
            h, i = int(spec["hidden_size"]), int(spec["intermediate_size"])
            out = [TensorDecl(f"{prefix}.router.weight", (int(spec["experts"]), h))]
            for e in range(int(spec["experts"])):
                out += [TensorDecl(f"{prefix}.experts.{e}.gate_proj.weight", (i, h)),
                        TensorDecl(f"{prefix}.experts.{e}.up_proj.weight", (i, h)),
                        TensorDecl(f"{prefix}.experts.{e}.down_proj.weight", (h, i))]
            return out

        def load(self, store, prefix, device):
            self.router = store.get(f"{prefix}.router.weight", torch.float32, device)
            self.w = [tuple(store.get(f"{prefix}.experts.{e}.{n}_proj.weight", torch.float32, device)
                            for n in ("gate", "up", "down")) for e in range(self.e)]

        def forward(self, x, ctx):
            xf = x.float()
            choice = kernels.gemm_tn(xf, self.router).argmax(dim=1)           # router logits in float32
            out = torch.zeros_like(xf)
            for e, (g, u, d) in enumerate(self.w):
                rows = (choice == e).nonzero().flatten()
                if rows.numel():
                    xe = xf[rows].contiguous()
                    a = kernels.silu_mul(torch.cat([kernels.gemm_tn(xe, g), kernels.gemm_tn(xe, u)], dim=1).contiguous())
                    out[rows] = kernels.gemm_tn(a, d)
            return out.to(self.dtype)

    @register_position_encoding("scaled_pairs")
    class ScaledPairs(PositionEncoding):
        """What the attention mixer reads of a position encoding: `cos` and `sin`
        [max_positions, rotary_dim / 2] float32, `rotary_dim`, `interleaved`."""

        def __init__(self, spec, dtype):
            super().__init__(spec, dtype)
            self.rotary_dim, self.interleaved = int(spec["rotary_dim"]), True
            self.theta, self.factor, self.max_positions = float(spec["theta"]), float(spec["factor"]), int(spec["max_positions"])
            self.cos = self.sin = None

        def load(self, store, prefix, device):
            inv = 1.0 / (self.theta ** (torch.arange(0, self.rotary_dim, 2, dtype=torch.float64) / self.rotary_dim))
            ang = (torch.arange(self.max_positions, dtype=torch.float64) / self.factor)[:, None] * inv[None, :]
            self.cos, self.sin = ang.cos().float().contiguous().to(device), ang.sin().float().contiguous().to(device)

    @dataclass(frozen=True)
    class ToyConfig:
        vocab_size: int
        architecture: str = "ToyRoutedForCausalLM"

        @classmethod
        def from_dict(cls, raw, where="config.json"):
            return cls(int(raw["vocab_size"]))

        def to_dict(self):
            return {"architectures": [self.architecture], "vocab_size": self.vocab_size}

    def toy_spec(cfg):
        norm = PartSpec("rmsnorm", dict(dim=H, eps=1e-5))
        pos = PartSpec("scaled_pairs", dict(rotary_dim=ROT, theta=THETA, factor=FACTOR, max_positions=256))
        attn = PartSpec("attention", dict(hidden_size=H, num_heads=3, num_kv_heads=1, head_dim=D, qk_norm=False,
                                          window=None, position=pos, scale=0.3))
        routed = PartSpec("top1_experts", dict(hidden_size=H, intermediate_size=I, experts=E))
        dense = PartSpec("gated_mlp", dict(hidden_size=H, intermediate_size=I, activation="silu"))
        norms = {"input_layernorm": norm, "post_attention_layernorm": norm}
        layers = (LayerSpec("model.layers.0", "prenorm", attn, routed, norms),
                  LayerSpec("model.layers.1", "prenorm", attn, dense, norms))
        return ModelSpec(
            architecture=cfg.architecture, vocab_size=cfg.vocab_size, hidden_size=H, max_positions=256,
            embedding=PartSpec("embedding", dict(name="model.embed_tokens.weight", vocab_size=cfg.vocab_size, dim=H)),
            layers=layers, schedule=(ScheduleEntry(0), ScheduleEntry(1)),
            final_norm=PartSpec("rmsnorm", dict(dim=H, eps=1e-5, name="model.norm.weight")),
            head=PartSpec("lm_head", dict(name="lm_head.weight", tied=False, vocab_size=cfg.vocab_size, dim=H)))

    register_architecture("ToyRoutedForCausalLM", ModelFamily("toy_routed", ToyConfig, toy_spec))
    d = write_random_model(str(tmp_path / "toy"), {"architectures": ["ToyRoutedForCausalLM"], "vocab_size": 61},
                           seed=5, linear_std=0.15)
    model = load_model(d, "float32", DEV)

    # the same model written out plainly, whole sequences, float64
    W = {k: v.double() for k, v in plain.read_weights(d).items()}
    inv = 1.0 / (THETA ** (torch.arange(0, ROT, 2, dtype=torch.float64) / ROT))

    def rotate(x, T):      # x [T, heads, D]: pairs (2i, 2i+1) of the first ROT dims, angle = p / FACTOR * inv[i]
        ang = (torch.arange(T, dtype=torch.float64) / FACTOR)[:, None] * inv[None, :]
        c, s = ang.cos()[:, None, :], ang.sin()[:, None, :]
        y = x.clone()
        a, b = x[..., 0:ROT:2], x[..., 1:ROT:2]
        y[..., 0:ROT:2], y[..., 1:ROT:2] = a * c - b * s, a * s + b * c
        return y

    used = set()

    def toy_logits(ids):
        T = len(ids)
        x = W["model.embed_tokens.weight"][torch.tensor(ids)]
        for i in range(2):
            p = f"model.layers.{i}"
            h = plain.rms_norm(x, W[f"{p}.input_layernorm.weight"], 1e-5)
            q = rotate((h @ W[f"{p}.self_attn.q_proj.weight"].T).reshape(T, 3, D), T)
            k = rotate((h @ W[f"{p}.self_attn.k_proj.weight"].T).reshape(T, 1, D), T)
            v = (h @ W[f"{p}.self_attn.v_proj.weight"].T).reshape(T, 1, D)
            r = x + plain.attention(q, k, v, scale=0.3).reshape(T, 3 * D) @ W[f"{p}.self_attn.o_proj.weight"].T
            h = plain.rms_norm(r, W[f"{p}.post_attention_layernorm.weight"], 1e-5)
            if i == 0:
                choice = (h @ W[f"{p}.mlp.router.weight"].T).argmax(dim=1)
                used.update(choice.tolist())
                m = torch.stack([plain.mlp_block(h[t:t + 1], W, f"{p}.mlp.experts.{int(choice[t])}")[0] for t in range(T)])
            else:
                m = plain.mlp_block(h, W, f"{p}.mlp")
            x = r + m
        return (plain.rms_norm(x, W["model.norm.weight"], 1e-5) @ W["lm_head.weight"].T).float()

    rng = random.Random(10)
    reqs = {f"q{i}": harness.random_prompt(rng, n, 61) for i, n in enumerate([23, 41, 9, 30])}
    ref = {rid: toy_logits(t) for rid, t in reqs.items()}
    assert used == set(range(E))           # every expert takes part
    for what, steps in (("whole", harness.trace_whole(reqs)), ("mixed", harness.trace_mixed(reqs, 1, max_live=2)),
                        ("portions", harness.trace_portions(reqs))):
        runner = ModelRunner(model, page_size=8, num_pages=14, max_requests=2)
        harness.compare(harness.replay(runner, steps), ref, harness.TOL["float32"], f"toy routed {what}")


# ---- a toy norm and a toy block arrangement, registered from here -----------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_norm_and_block_arrangement(dtype, tmp_path):
    """Two more part kinds defined in this test: a norm that centres its rows and has a bias
    (nothing a product could carry, so it is not foldable), and a block arrangement in which the
    mixer and the feed-forward read the same normed rows and their sum goes through a second norm
    before it joins the stream.  The architecture runs a built-in "prenorm" layer, the toy
    arrangement, and the prenorm layer again (so a block that folds norms runs before and after
    one that does not), and ends in the toy norm as its final norm (which norms the wanted rows
    only).  Registered, written, loaded and stepped in every way of cutting, without a change to
    the framework's files."""
    from dataclasses import dataclass
    from xinfer_amd.config.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry
    from xinfer_amd.engine import ModelRunner, load_model
    from xinfer_amd.models import ModelFamily, register_architecture
    from xinfer_amd.parts import (Block, Norm, Stream, feed_forward_class, mixer_class, norm_class, register_block,
                                  register_norm)
    from xinfer_amd.weights import TensorDecl, write_random_model

    H, D, V, EPS = 48, 16, 83, 3e-4

    @register_norm("centered")
    class Centered(Norm):
        """out = (s - mean(s)) * rsqrt(var(s) + eps) * weight + bias, s = resid (+ add), in float32.  The
        contract of a norm: without `rows` the sum is written back into `resid` and every row is
        normed; with `rows` only those rows are made and `resid` is left alone; `add` may be a stack
        [P, T, H] of float32 partial sums."""

        def __init__(self, spec, dtype):
            super().__init__(spec, dtype)
            self.dim, self.eps = int(spec["dim"]), float(spec["eps"])

        @classmethod
        def declare(cls, spec, prefix):
            return [TensorDecl(f"{prefix}.weight", (int(spec["dim"]),), "norm"), TensorDecl(f"{prefix}.bias", (int(spec["dim"]),))]

        def load(self, store, prefix, device):
            self.weight = store.get(f"{prefix}.weight", torch.float32, device)
            self.bias = store.get(f"{prefix}.bias", torch.float32, device)

        def forward(self, resid, add, out_dtype, rows=None, out=None):
            if add is not None:
                add = add.sum(0) if add.dim() == 3 else add.float()
            if rows is None:
                if add is not None:
                    resid += add
                s = resid
            else:
                s = resid[rows.long()] + (add[rows.long()] if add is not None else 0.0)
            c = s - s.mean(1, keepdim=True)
            y = (c * torch.rsqrt((c * c).mean(1, keepdim=True) + self.eps) * self.weight + self.bias).to(out_dtype)
            if out is not None:
                out.copy_(y)
                return out
            return y

    @register_block("parallel_then_norm")
    class ParallelThenNorm(Block):
        """r = x + norm_b(mixer(norm_a(x)) + feed_forward(norm_a(x)))"""

        def __init__(self, layer, dtype):
            super().__init__(layer, dtype)
            self.mixer = mixer_class(layer.mixer.kind)(layer.mixer, dtype)
            self.ffn = feed_forward_class(layer.feed_forward.kind)(layer.feed_forward, dtype)
            (self.name_a, a), (self.name_b, b) = layer.norm_items(2)
            self.norm_a, self.norm_b = norm_class(a.kind)(a, dtype), norm_class(b.kind)(b, dtype)

        @classmethod
        def declare(cls, layer):
            p = layer.prefix
            out = mixer_class(layer.mixer.kind).declare(layer.mixer, f"{p}.{layer.mixer_name}")
            out += feed_forward_class(layer.feed_forward.kind).declare(layer.feed_forward, f"{p}.{layer.feed_forward_name}")
            for name, n in layer.norm_items(2):
                out += norm_class(n.kind).declare(n, f"{p}.{name}")
            return out

        def load(self, store, device):
            p = self.layer.prefix
            self.mixer.load(store, f"{p}.{self.layer.mixer_name}", device)
            self.ffn.load(store, f"{p}.{self.layer.feed_forward_name}", device)
            self.norm_a.load(store, f"{p}.{self.name_a}", device)
            self.norm_b.load(store, f"{p}.{self.name_b}", device)

        def cache_need(self):
            return self.mixer.cache_need()

        def forward(self, stream, ctx, cache):
            def whole(y):                    # a part may answer with a stack of float32 partial sums
                return y.sum(0) if y.dim() == 3 else y.float()
            h = self.norm_a.forward(stream.resid, stream.pending, self.dtype)
            branch = (whole(self.mixer.forward(h, ctx, cache)) + whole(self.ffn.forward(h, ctx))).contiguous()
            return Stream(stream.resid, self.norm_b.forward(branch, None, torch.float32))

    @dataclass(frozen=True)
    class ToyConfig:
        vocab_size: int
        architecture: str = "ToyParallelForCausalLM"

        @classmethod
        def from_dict(cls, raw, where="config.json"):
            return cls(int(raw["vocab_size"]))

        def to_dict(self):
            return {"architectures": [self.architecture], "vocab_size": self.vocab_size}

    def toy_spec(cfg):
        rms = PartSpec("rmsnorm", dict(dim=H, eps=1e-5))
        cen = PartSpec("centered", dict(dim=H, eps=EPS))
        rope = PartSpec("rope", dict(head_dim=D, rotary_dim=D, theta=10000.0, max_positions=256))
        attn = PartSpec("attention", dict(hidden_size=H, num_heads=3, num_kv_heads=1, head_dim=D, qk_norm=True, qk_norm_eps=1e-5,
                                          window=None, position=rope, scale=0.25))
        ffn = PartSpec("gated_mlp", dict(hidden_size=H, intermediate_size=80, activation="silu"))
        layers = (LayerSpec("model.layers.0", "prenorm", attn, ffn, {"input_layernorm": rms, "post_attention_layernorm": rms}),
                  LayerSpec("model.layers.1", "parallel_then_norm", attn, ffn, {"ln_in": cen, "ln_out": rms}))
        return ModelSpec(
            architecture=cfg.architecture, vocab_size=cfg.vocab_size, hidden_size=H, max_positions=256,
            embedding=PartSpec("embedding", dict(name="model.embed_tokens.weight", vocab_size=cfg.vocab_size, dim=H)),
            # the prenorm layer runs again after the toy arrangement and reads the cache of its first run
            layers=layers, schedule=(ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(0, cache_of=0)),
            final_norm=PartSpec("centered", dict(dim=H, eps=EPS, prefix="model.norm")),
            head=PartSpec("lm_head", dict(name="lm_head.weight", tied=False, vocab_size=cfg.vocab_size, dim=H)))

    register_architecture("ToyParallelForCausalLM", ModelFamily("toy_parallel", ToyConfig, toy_spec))
    d = write_random_model(str(tmp_path / "toy"), {"architectures": ["ToyParallelForCausalLM"], "vocab_size": V},
                           seed=6, linear_std=0.15)
    model = load_model(d, dtype, DEV)
    assert not model.blocks[1].graph_safe and model.blocks[0].graph_safe

    W = plain.read_weights(d)
    cos, sin = plain.rope_tables(10000.0, D, 256)

    def centered(x, name):
        c = x - x.mean(1, keepdim=True)
        return c / torch.sqrt((c * c).mean(1, keepdim=True) + EPS) * W[f"{name}.weight"] + W[f"{name}.bias"]

    def qkv(h, p, T):
        def heads(name, n, norm):
            y = (h @ W[f"{p}.{name}_proj.weight"].T).reshape(T, n, D)
            return plain.apply_rope(plain.rms_norm(y, W[f"{p}.{norm}.weight"], 1e-5), torch.arange(T), cos, sin) if norm else y
        return heads("q", 3, "q_norm"), heads("k", 1, "k_norm"), heads("v", 1, None)

    def toy_logits(ids):
        T = len(ids)
        x = W["model.embed_tokens.weight"][torch.tensor(ids)]
        kv = None
        for run in (0, 1, 2):
            if run == 1:
                p = "model.layers.1"
                h = centered(x, f"{p}.ln_in")
                q, k, v = qkv(h, f"{p}.self_attn", T)
                a = plain.attention(q, k, v, scale=0.25).reshape(T, 3 * D) @ W[f"{p}.self_attn.o_proj.weight"].T
                x = x + plain.rms_norm(a + plain.mlp_block(h, W, f"{p}.mlp"), W[f"{p}.ln_out.weight"], 1e-5)
                continue
            p = "model.layers.0"
            h = plain.rms_norm(x, W[f"{p}.input_layernorm.weight"], 1e-5)
            q, k, v = qkv(h, f"{p}.self_attn", T)
            if kv is None:
                kv = (k, v)
            r = x + plain.attention(q, kv[0], kv[1], scale=0.25).reshape(T, 3 * D) @ W[f"{p}.self_attn.o_proj.weight"].T
            x = r + plain.mlp_block(plain.rms_norm(r, W[f"{p}.post_attention_layernorm.weight"], 1e-5), W, f"{p}.mlp")
        return centered(x, "model.norm") @ W["lm_head.weight"].T

    rng = random.Random(12)
    reqs = {f"q{i}": harness.random_prompt(rng, n, V) for i, n in enumerate([27, 50, 6, 38])}
    ref = {rid: toy_logits(t) for rid, t in reqs.items()}
    for what, steps in (("whole", harness.trace_whole(reqs)), ("mixed", harness.trace_mixed(reqs, 1, max_live=2)),
                        ("portions", harness.trace_portions(reqs)), ("tail", harness.trace_tail_one_by_one(reqs, tail=20))):
        runner = ModelRunner(model, page_size=8, num_pages=harness.tokens_needed(steps, 8) // 8, max_requests=2)
        harness.compare(harness.replay(runner, steps), ref, harness.TOL[dtype], f"toy parallel {dtype} {what}")


# ---- the measurement script -------------------------------------------------------------------------------
def test_bench_line_keeps_its_contract():
    """`bench.py` with two layers: one JSON line with the contract's fields, a flat `config` of at
    most 20 keys that names both layer counts, the prefill and roofline records and the two points."""
    import json
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--layers", "2", "--steps", "4", "--warmup", "1"],
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "prefill", "roofline", "points"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 4 and d["warmup"] == 1 and d["higher_is_better"] is True
    assert d["value"] > 0 and abs(d["value"] - 8 / (d["ms_per_step"] / 1e3)) / d["value"] < 1e-3
    cfg = d["config"]
    assert len(cfg) <= 20 and all(not isinstance(v, (dict, list)) for v in cfg.values())
    assert cfg["layers"] == 2 and cfg["layers_of_model"] == 36 and cfg["global_batch"] == 8 and cfg["seq_len"] == 4096
    assert set(d["prefill"]) == {"value", "tokens", "ms", "frac"} and d["prefill"]["tokens"] == 2048
    assert d["roofline"]["bound"] == "hbm" and d["roofline"]["peak"] == 8000.0 and d["roofline"]["unit"] == "GB/s"
    assert abs(d["roofline"]["frac"] - d["roofline"]["achieved"] / 8000.0) < 1e-3
    assert set(d["points"]) == {"decode_b1", "decode_b64"} == set(d["points_roofline"])
    for name, r in d["points_roofline"].items():
        batch = int(name.split("_b")[1])
        assert abs(r["frac"] - r["achieved"] / 8000.0) < 1e-3 and abs(batch / (r["ms_per_step"] / 1e3) / d["points"][name] - 1) < 1e-3
    assert d["further"]["decode_b8_ctx"] == 16384 and d["further"]["frac"] > 0
