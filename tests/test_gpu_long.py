"""Contexts of some thousand keys, at model level against the plain implementation and at kernel
level on the cases of the reference's own attention probe: prompt portions that attend to a
cached prefix of 2,048 and of 4,096 keys and more, single-token steps replayed from graphs while
the context crosses 4,096 (another graph bucket, other keys per workgroup, the wide combine of
the split-K decode kernel), and decode batches of requests of unequal lengths."""
import math
import random

import pytest
import torch

import harness
import plain_qwen3 as plain
from configs import LONG

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = ["float32", "bfloat16"]


@pytest.fixture(scope="module")
def long_model(tmp_path_factory):
    """The LONG model folder (q_norm weights multiplied by `sharpen`) and the plain model of it."""
    from safetensors.torch import load_file, save_file
    from xinfer_amd.weights import write_random_model
    d = str(tmp_path_factory.mktemp("long_model"))
    write_random_model(d, LONG["config"], LONG["seed"], LONG["linear_std"], LONG["norm_std"])
    path = d + "/model.safetensors"
    tensors = load_file(path)
    for name in tensors:
        if name.endswith("q_norm.weight"):
            tensors[name] = (tensors[name].float() * LONG["sharpen"]).to(tensors[name].dtype)
    save_file(tensors, path)
    return d, plain.PlainModel(d)


def _softmax_is_sharp(pm, ids):
    """The share of the largest weight in the last row's softmax of layer 0, head 0 (a check of the
    test's own construction: the rows must not be flat averages)."""
    c, W = pm.config, pm.weights
    cos, sin = plain.rope_tables(float(c["rope_theta"]), c["head_dim"], c["max_position_embeddings"])
    x = W["model.embed_tokens.weight"][torch.tensor(ids)]
    h = plain.rms_norm(x, W["model.layers.0.input_layernorm.weight"], c["rms_norm_eps"])
    T, d = len(ids), c["head_dim"]
    pos = torch.arange(T)
    q = (h @ W["model.layers.0.self_attn.q_proj.weight"].T).reshape(T, -1, d)[:, :1]
    k = (h @ W["model.layers.0.self_attn.k_proj.weight"].T).reshape(T, -1, d)[:, :1]
    q = plain.apply_rope(plain.rms_norm(q, W["model.layers.0.self_attn.q_norm.weight"], c["rms_norm_eps"]), pos, cos, sin)
    k = plain.apply_rope(plain.rms_norm(k, W["model.layers.0.self_attn.k_norm.weight"], c["rms_norm_eps"]), pos, cos, sin)
    s = (q[-1, 0] @ k[:, 0].T) / math.sqrt(d)
    return float(torch.softmax(s, dim=-1).max())


_refs = {}


def _ref(pm, reqs):
    """Plain logits of the requests; a request that is the beginning of one already computed takes
    the beginning of its logits (the model is causal)."""
    out = {}
    for rid, toks in reqs.items():
        key = tuple(toks)
        hit = next((k for k in _refs if k[:len(key)] == key), None)
        if hit is None:
            _refs[key] = pm.logits(toks)
            hit = key
        out[rid] = _refs[hit][:len(toks)]
    return out


def _one_long_request():
    rng = random.Random(41)
    return {"long": harness.random_prompt(rng, 6200, LONG["config"]["vocab_size"])}


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_request_portions_and_decoding_across_4096(dtype, long_model):
    """One request of 6,200 tokens: portions of 2,048 and 2,000 (the second attends to 2,048 cached
    keys), 60 single tokens from 4,048 to 4,108 (recorded the third time a bucket is seen and replayed
    from then on: the bucket of 4,096 keys, then the one of 5,120), a portion of 2,048 behind 4,108
    cached keys, and single tokens to the end (the bucket of 7,168); every position's logits against the plain model."""
    from xinfer_amd.engine import ModelRunner, load_model
    d, pm = long_model
    reqs = _one_long_request()
    toks = reqs["long"]
    assert _softmax_is_sharp(pm, toks[:4200]) > 8 / 4200         # flat would be 1 / 4200
    cuts = [2048, 2000] + [1] * 60 + [2048] + [1] * (6200 - 4108 - 2048)
    assert sum(cuts) == len(toks)
    steps, p = [], 0
    for i, n in enumerate(cuts):
        steps.append({"step": i, "entries": [{"id": "long", "tokens": toks[p:p + n], "want": list(range(n))}],
                      "end": ["long"] if p + n == len(toks) else []})
        p += n
    page = LONG["page_size"]
    model = load_model(d, dtype, DEV)
    runner = ModelRunner(model, page_size=page, num_pages=-(-len(toks) // page), max_requests=2, graph_after=3)
    got = harness.replay(runner, steps)
    assert len(got) == len(toks)
    assert {k[1] for k in runner._graphs} == {4096, 5120, 7168} and runner.graph_replays >= 60
    rel = harness.compare(got, _ref(pm, reqs), harness.TOL[dtype], f"LONG/{dtype}/one request")
    print(f"LONG/{dtype}/one request: worst error {rel:.2e} of the largest logit")


@pytest.mark.parametrize("dtype", DTYPES)
def test_decode_batch_of_eight_unequal_lengths(dtype, long_model):
    """Eight requests of 1,500 to 6,000 tokens: their heads as portions of 2,048 tokens a step (the
    later portions of a request beside the first of the next), then six steps that bring one token of
    each: launched twice, then recorded and replayed."""
    from xinfer_amd.engine import ModelRunner, load_model
    d, pm = long_model
    rng = random.Random(43)
    lens = [1500, 1800, 2100, 2600, 3300, 4090, 4700, 6000]
    reqs = {f"r{i}": harness.random_prompt(rng, n, LONG["config"]["vocab_size"]) for i, n in enumerate(lens)}
    reqs["r7"] = _one_long_request()["long"][:lens[7]]         # the beginning of the other test's request
    tail = 6
    steps, budget = [], 2048
    pos = {rid: 0 for rid in reqs}
    order = list(reqs)
    while any(pos[r] < len(reqs[r]) - tail for r in order):
        entries, left = [], budget
        for r in order:
            n = min(left, len(reqs[r]) - tail - pos[r])
            if n > 0:
                entries.append({"id": r, "tokens": reqs[r][pos[r]:pos[r] + n], "want": list(range(max(0, n - 3), n))})
                pos[r] += n
                left -= n
        steps.append({"step": len(steps), "entries": entries, "end": []})
    for k in range(tail):
        steps.append({"step": len(steps), "end": order if k == tail - 1 else [], "entries": [
            {"id": r, "tokens": [reqs[r][len(reqs[r]) - tail + k]], "want": [0]} for r in order]})
    page = LONG["page_size"]
    model = load_model(d, dtype, DEV)
    runner = ModelRunner(model, page_size=page, num_pages=sum(-(-n // page) for n in lens), max_requests=8, graph_after=3)
    got = harness.replay(runner, steps)
    assert runner.graph_replays == tail - 3 and list(runner._graphs) == [(8, 6144, False)]
    rel = harness.compare(got, _ref(pm, reqs), harness.TOL[dtype], f"LONG/{dtype}/batch of eight")
    print(f"LONG/{dtype}/batch of eight: worst error {rel:.2e} of the largest logit")


# ---- the matrix-core attention kernels against the generic kernel, inside the model ---------------------------
_long_dirs = {}


def _long_dir(tmp_path_factory, sharpen):
    """The LONG model folder with its q_norm weights multiplied by `sharpen`."""
    from safetensors.torch import load_file, save_file
    from xinfer_amd.weights import write_random_model
    if sharpen not in _long_dirs:
        d = str(tmp_path_factory.mktemp(f"long_model_{sharpen}"))
        write_random_model(d, LONG["config"], LONG["seed"], LONG["linear_std"], LONG["norm_std"])
        tensors = load_file(d + "/model.safetensors")
        for name in tensors:
            if name.endswith("q_norm.weight"):
                tensors[name] = (tensors[name].float() * sharpen).to(tensors[name].dtype)
        save_file(tensors, d + "/model.safetensors")
        _long_dirs[sharpen] = d
    return _long_dirs[sharpen]


def _long_steps():
    """The long request's steps (portions behind 0, 2,048 and 4,108 cached keys, single tokens across
    4,096 and to the end) and eight requests of unequal lengths whose last six tokens come together."""
    toks = _one_long_request()["long"]
    cuts = [2048, 2000] + [1] * 60 + [2048] + [1] * (6200 - 4108 - 2048)
    steps, p = [], 0
    for n in cuts:
        steps.append({"step": len(steps), "entries": [{"id": "long", "tokens": toks[p:p + n], "want": list(range(max(0, n - 4), n))}],
                      "end": ["long"] if p + n == len(toks) else []})
        p += n
    rng = random.Random(47)
    reqs = {f"r{i}": harness.random_prompt(rng, n, LONG["config"]["vocab_size"]) for i, n in enumerate([900, 1500, 2100, 2600, 3300, 4090, 4700, 5800])}
    tail, pos = 6, {r: 0 for r in reqs}
    while any(pos[r] < len(reqs[r]) - tail for r in reqs):
        entries, left = [], 2048
        for r in reqs:
            n = min(left, len(reqs[r]) - tail - pos[r])
            if n > 0:
                entries.append({"id": r, "tokens": reqs[r][pos[r]:pos[r] + n], "want": list(range(max(0, n - 2), n))})
                pos[r] += n
                left -= n
        steps.append({"step": len(steps), "entries": entries, "end": []})
    for k in range(tail):
        steps.append({"step": len(steps), "end": list(reqs) if k == tail - 1 else [], "entries": [
            {"id": r, "tokens": [reqs[r][len(reqs[r]) - tail + k]], "want": [0]} for r in reqs]})
    return steps


@pytest.mark.parametrize("sharpen", [1.5, 3.0])
def test_matrix_core_attention_agrees_with_the_generic_kernel_inside_the_model(sharpen, tmp_path_factory):
    """Inside the bfloat16 model, as the engine runs it (runner, graphs, context buckets, the ring
    prefill kernel, the split-K decode kernel that norms, rotates and stores its own heads), every
    attention call is followed by the generic kernel (one thread a score, float32 softmax weights,
    no matrix cores; the float32 tests hold it against the plain model) on the very same q and
    cache, and the two outputs are compared.  The inputs are the same bits, so what is left is
    the kernels' own: the matrix-core kernels round the softmax weights to bfloat16 before the
    second product (at most 2^-9 of the largest |v|), both round their output to bfloat16 (2^-9 of
    it each), sums are taken in other orders: less than 2^-7 of the largest |v| together, at any
    sharpness of the scores; a key dropped or misplaced moves a row by its weight times |v|.
    Logit-level comparisons cannot separate this: one flipped rounding of an activation grows
    through the layers like any other rounding error."""
    from xinfer_amd import kernels
    from xinfer_amd.engine import ModelRunner, load_model
    d = _long_dir(tmp_path_factory, sharpen)
    page = LONG["page_size"]
    steps = _long_steps()
    pages = harness.tokens_needed(steps, page) // page
    model = load_model(d, "bfloat16", DEV)
    worst = torch.zeros(2, dtype=torch.float32, device=DEV)       # [largest |difference| / largest |v|, calls]
    one = torch.ones((), dtype=torch.float32, device=DEV)

    def note(a, ref, v_cache):
        ratio = (a.float() - ref.float()).abs().max() / v_cache.float().abs().max()
        worst[0].copy_(torch.maximum(worst[0], ratio))             # device work only: it is recorded into the graphs too
        worst[1].add_(one)

    inner_attention, inner_packed = kernels.attention, kernels.attention_decode_packed_bf16

    def attention(q, k_cache, v_cache, ctx, group, scale, window=0, v_grouped=False):
        a = inner_attention(q, k_cache, v_cache, ctx, group, scale, window, v_grouped=v_grouped)
        note(a, kernels.attention_generic(q, k_cache, v_cache, ctx.block_tables[group], ctx.tok_seq, ctx.positions, scale,
                                          window, v_grouped=v_grouped), v_cache)
        return a

    def packed(qkv, q_weight, k_weight, eps, cos, sin, rotary_dim, interleaved, positions, slots, k_cache, vt_cache,
               block_tables, ctx_lens, max_ctx_len, num_heads, scale, window=0, bias=None, similar=False):
        a = inner_packed(qkv, q_weight, k_weight, eps, cos, sin, rotary_dim, interleaved, positions, slots, k_cache, vt_cache,
                         block_tables, ctx_lens, max_ctx_len, num_heads, scale, window, bias=bias, similar=similar)
        # the heads as the stand-alone kernel norms and rotates them (it stores nothing: every slot is -1);
        # the new keys and values are in the cache already, written by the kernel under test
        B = positions.shape[0]
        q = kernels.qk_norm_rope_kv(qkv, q_weight, k_weight, eps, cos, sin, rotary_dim, interleaved, positions,
                                    torch.full((B,), -1, dtype=torch.int64, device=DEV), k_cache, vt_cache, num_heads,
                                    k_cache.shape[1], k_cache.shape[3], v_grouped=True, vector_min_tokens=1 << 30, bias=bias)
        note(a, kernels.attention_generic(q, k_cache, vt_cache, block_tables, torch.arange(B, dtype=torch.int32, device=DEV),
                                          positions, scale, window, v_grouped=True), vt_cache)
        return a

    kernels.attention, kernels.attention_decode_packed_bf16 = attention, packed
    try:
        runner = ModelRunner(model, page_size=page, num_pages=pages, max_requests=8, graph_after=3)
        got = harness.replay(runner, steps)
    finally:
        kernels.attention, kernels.attention_decode_packed_bf16 = inner_attention, inner_packed
    assert runner.graph_replays > 60 and got
    ratio, calls = worst.tolist()
    layers = len(model.blocks)
    assert calls == layers * len(steps)                             # replays counted too: the check is part of the graph
    print(f"LONG/bfloat16/sharpen {sharpen}: over {int(calls)} attention calls the matrix-core kernels differ from the "
          f"generic one by at most {ratio:.2e} of the largest |v|")
    assert ratio < 2.0 ** -7


@pytest.mark.parametrize("dtype", DTYPES)
def test_decode_batch_of_eight_equal_lengths_at_4096(dtype, long_model):
    """Eight requests of 4,082 to 4,096 tokens decode their last twelve tokens together: sequences
    about equally long, recorded at the third step for the bucket of 4,096 keys (four splits of
    1,024 keys a sequence) and replayed nine times; against the plain model."""
    from xinfer_amd.engine import ModelRunner, load_model
    d, pm = long_model
    rng = random.Random(53)
    base = [_one_long_request()["long"], harness.random_prompt(rng, 4096, LONG["config"]["vocab_size"])]
    reqs = {f"e{i}": base[i % 2][:4096 - 2 * i] for i in range(8)}
    tail, budget = 12, 2048
    steps, pos = [], {r: 0 for r in reqs}
    while any(pos[r] < len(reqs[r]) - tail for r in reqs):
        entries, left = [], budget
        for r in reqs:
            n = min(left, len(reqs[r]) - tail - pos[r])
            if n > 0:
                entries.append({"id": r, "tokens": reqs[r][pos[r]:pos[r] + n], "want": [n - 1]})
                pos[r] += n
                left -= n
        steps.append({"step": len(steps), "entries": entries, "end": []})
    for k in range(tail):
        steps.append({"step": len(steps), "end": list(reqs) if k == tail - 1 else [], "entries": [
            {"id": r, "tokens": [reqs[r][len(reqs[r]) - tail + k]], "want": [0]} for r in reqs]})
    page = LONG["page_size"]
    runner = ModelRunner(load_model(d, dtype, DEV), page_size=page, num_pages=8 * (4096 // page), max_requests=8, graph_after=3)
    got = harness.replay(runner, steps)
    assert list(runner._graphs) == [(8, 4096, True)] and runner.graph_replays == tail - 3
    rel = harness.compare(got, _ref(pm, reqs), harness.TOL[dtype], f"LONG/{dtype}/eight of equal length")
    print(f"LONG/{dtype}/eight of equal length: worst error {rel:.2e} of the largest logit")


# ---- the reference's attention probe cases --------------------------------------------------------
def _rows_golden(q, q_pos, k, v, scale):
    """Dense float32 attention of the query rows alone: q [n, hq, d] at absolute positions q_pos
    over k, v [kv_len, hkv, d]; contiguous groups of query heads share a kv head; keys behind a
    query's position are masked.  /root/reference/tests/probes/compare_flashinfer_probe.py:51-73."""
    n, hq, d = q.shape
    hkv = k.shape[1]
    g = hq // hkv
    kpos = torch.arange(k.shape[0])
    out = torch.empty((n, hq, d), dtype=torch.float32)
    for h in range(hq):
        s = (q[:, h].float() @ k[:, h // g].float().T) * scale
        s = s.masked_fill(kpos[None, :] > q_pos[:, None], float("-inf"))
        out[:, h] = torch.softmax(s, dim=-1) @ v[:, h // g].float()
    return out


PROBE_CASES = [            # (prefix, append, hq, hkv): flashinfer_precision_probe.rs:205-295, d = 128, page = 64
    (0, 1024, 8, 2), (65, 257, 8, 2), (4097, 257, 8, 2), (32769, 257, 8, 2), (65536, 64, 32, 4)]


@pytest.mark.parametrize("page_map", ["plus3", "shuffled"])
@pytest.mark.parametrize("prefix,append,hq,hkv", PROBE_CASES)
def test_reference_attention_probe_cases(prefix, append, hq, hkv, page_map):
    """The cases of the reference's paged-prefill probe (flashinfer_precision_probe.rs:33-196): q, k, v
    ~ N(0, 1) in bfloat16, the prefix laid into the pages, the appended keys and values written by
    the cache-write kernel, the appended queries attend causally to prefix + append; pages i + 3 as
    there, and shuffled.  Against the dense float32 golden of the queried rows with the probe's
    absolute tolerance 0.015625 (compare_flashinfer_probe.py:154-165), and, since rows that
    average tens of thousands of values are smaller than that themselves, also relative to the
    largest value of each (row, head).  The last four positions then go through the split-K decode kernel as four
    sequences that share the pages, and one far key is made to win a row's softmax."""
    from xinfer_amd import kernels
    d, page = 128, 64
    scale = 1.0 / math.sqrt(d)
    g = torch.Generator().manual_seed(prefix + append)
    kv_len = prefix + append
    n_pages = -(-kv_len // page)
    k = torch.randn((kv_len, hkv, d), generator=g).to(torch.bfloat16)
    v = torch.randn((kv_len, hkv, d), generator=g).to(torch.bfloat16)
    q = torch.randn((append, hq, d), generator=g).to(torch.bfloat16)
    far = max(0, prefix - 2)                   # in the prefix's last, partly filled page (or the first key)
    grp = hq // hkv
    for j in range(hkv):                       # the last query's first head of every group points at key `far`
        k[far, j] = (q[-1, j * grp].float() / q[-1, j * grp].float().norm() * 60).to(torch.bfloat16)
    if page_map == "plus3":
        phys = [i + 3 for i in range(n_pages)]
    else:
        phys = (torch.randperm(n_pages + 3, generator=g)[:n_pages]).tolist()
    kc = torch.zeros((n_pages + 3, hkv, page, d), dtype=torch.bfloat16)
    vc = torch.zeros((n_pages + 3, hkv, page, d), dtype=torch.bfloat16)
    for lp in range(-(-prefix // page)):
        n = min(page, prefix - lp * page)
        kc[phys[lp], :, :n] = k[lp * page:lp * page + n].transpose(0, 1)
        vc[phys[lp], :, :n] = v[lp * page:lp * page + n].transpose(0, 1)
    # the bfloat16 path keeps V in groups of eight keys: [pages, kv heads, page / 8, d, 8]
    vt = vc.reshape(n_pages + 3, hkv, page // 8, 8, d).transpose(3, 4).contiguous()
    kc, vt = kc.to(DEV), vt.to(DEV)
    bt = torch.tensor([phys], dtype=torch.int32, device=DEV)
    positions = torch.arange(prefix, kv_len, dtype=torch.int32)
    slots = torch.tensor([phys[p // page] * page + p % page for p in range(prefix, kv_len)], dtype=torch.int64)
    packed = torch.cat([q.reshape(append, -1), k[prefix:].reshape(append, -1), v[prefix:].reshape(append, -1)], dim=1)
    none = torch.empty((1, 0), dtype=torch.float32, device=DEV)
    q_dev = kernels.qk_norm_rope_kv(packed.contiguous().to(DEV), None, None, 1e-6, none, none, 0, False,
                                    positions.to(DEV), slots.to(DEV), kc, vt, hq, hkv, d, v_grouped=True)
    assert torch.equal(q_dev.cpu(), q)
    # the pages read back through the table hold k and v in order (compare_flashinfer_probe.py:102-113)
    idx = torch.tensor(phys, device=DEV)
    assert torch.equal(kc[idx].permute(0, 2, 1, 3).reshape(-1, hkv, d)[:kv_len].cpu(), k)
    assert torch.equal(vt[idx].transpose(3, 4).reshape(len(phys), hkv, page, d).permute(0, 2, 1, 3).reshape(-1, hkv, d)[:kv_len].cpu(), v)

    gold = _rows_golden(q, positions.long(), k, v, scale)
    assert (gold[-1, 0] - v[far, 0].float()).abs().max() < 0.05            # the far key won that row

    def check(out, rows, what):
        err = (out.float().cpu().reshape(-1, hq, d) - gold[rows]).abs()
        assert float(err.max()) <= 0.015625, (what, float(err.max()))
        rel = err.amax(dim=2) / gold[rows].abs().amax(dim=2)          # per (row, head), of its largest value
        assert float(rel.max()) < 2.0 ** -7, (what, float(rel.max()))

    cu = torch.tensor([0, append], dtype=torch.int32, device=DEV)
    cl = torch.tensor([kv_len], dtype=torch.int32, device=DEV)
    for small in (0, 1, 2):           # every workgroup shape of the prefill kernel
        qb = kernels.prefill_block(d, grp, small)
        tiles = torch.tensor([(0, q0) for q0 in range(0, append, qb)], dtype=torch.int32, device=DEV)
        out = kernels.attention_prefill_bf16(q_dev, kc, vt, bt, tiles, cu, cl, scale, 0, small=small)
        check(out, slice(None), f"prefill small={small}")
    from xinfer_amd.engine.runner import context_bucket
    n_last = min(4, append)
    lens = torch.arange(kv_len - n_last + 1, kv_len + 1, dtype=torch.int32, device=DEV)
    bucket = max(context_bucket(kv_len), 2 * kv_len)     # a recorded step's grid is laid out for more keys than there are: here twice
    wide = torch.zeros((n_last, -(-bucket // page)), dtype=torch.int32, device=DEV)
    wide[:, :n_pages] = bt
    for kpw, span, tables, similar in ((None, kv_len, bt.expand(n_last, -1).contiguous(), False), (128, kv_len, wide, False),
                                       (None, bucket, wide, False), (None, context_bucket(kv_len), wide, True)):
        out = kernels.attention_decode_bf16(q_dev[-n_last:].contiguous(), kc, vt, tables, lens, span, scale, 0,
                                            keys_per_workgroup=kpw, similar=similar)
        check(out, slice(append - n_last, append), f"decode kpw={kpw} span={span} similar={similar}")
    out = kernels.attention_generic(q_dev[-n_last:].contiguous(), kc, vt, bt, torch.zeros(n_last, dtype=torch.int32, device=DEV),
                                    positions[-n_last:].to(DEV), scale, 0, v_grouped=True)
    check(out, slice(append - n_last, append), "generic")
