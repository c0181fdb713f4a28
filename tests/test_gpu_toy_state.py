"""Two toy parts registered from here, for what the step function owes parts of other kinds: a
mixer whose per-request state lives and is updated on the device alone, so that it may be
recorded into a decode graph, and an embedding that reads the step's positions.

The reference records exact batch sizes because of such state slots
(/root/reference/src/utils/graph.rs:415-420: replaying a graph of a hybrid model needs the
batch it was recorded for); here the concern is that every step, the one that records a
graph too, advances the state exactly once."""
import random
from dataclasses import dataclass

import pytest
import torch

import harness
import plain_qwen3 as plain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

H, D, V, DECAY, POSITIONS = 32, 16, 89, 0.75, 160


def _register():
    from xinfer_amd import kernels
    from xinfer_amd.config.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry
    from xinfer_amd.models import ModelFamily, register_architecture
    from xinfer_amd.parts import Mixer, StateNeed, TokenEmbedding, register_embedding, register_mixer
    from xinfer_amd.weights import TensorDecl

    @register_mixer("decayed_sum")
    class DecayedSum(Mixer):
        """s[t] = decay * s[t-1] + x[t] per request, y[t] = W s[t].  The state slot holds s; every
        read and write of it is an index operation on `ctx.state_slots`, and the scan over a
        portion's tokens is one product with a [T, T] matrix made from `tok_seq` and `positions`
        on the device: nothing of the step is read on the host."""
        graph_safe = True

        def __init__(self, spec, dtype):
            super().__init__(spec, dtype)
            self.h, self.decay = int(spec["hidden_size"]), float(spec["decay"])

        @classmethod
        def declare(cls, spec, prefix):
            return [TensorDecl(f"{prefix}.mix.weight", (int(spec["hidden_size"]),) * 2)]

        def load(self, store, prefix, device):
            self.w = store.get(f"{prefix}.mix.weight", torch.float32, device)

        def state_need(self):
            return StateNeed((self.h,), torch.float32)

        def forward(self, x, ctx, cache):
            seq = ctx.tok_seq.long()
            pos = ctx.positions.long()
            slots = ctx.state_slots.index_select(0, seq)                        # [T]
            first = pos - (torch.arange(ctx.num_tokens, device=x.device) - ctx.cu_q.long().index_select(0, seq))
            before = cache.state.index_select(0, slots)                          # the state each token's request came with
            gap = pos[:, None] - pos[None, :]
            same = (seq[:, None] == seq[None, :]) & (gap >= 0)
            m = torch.where(same, torch.pow(self.decay, gap.clamp(min=0).float()), torch.zeros((), device=x.device))
            s = kernels.gemm_tn(m.contiguous(), x.float().t().contiguous())
            s = s + before * torch.pow(self.decay, (pos - first + 1).float())[:, None]
            last = ctx.cu_q.long()[1:] - 1                                       # each request's last token of the step
            cache.state.index_copy_(0, ctx.state_slots, s.index_select(0, last))
            return kernels.gemm_tn(s.contiguous(), self.w).to(self.dtype)

    @register_embedding("embedding_with_positions")
    class EmbeddingWithPositions(TokenEmbedding):
        """x = E[id] + P[position]: an embedding that needs the step."""
        graph_safe = True

        @classmethod
        def declare(cls, spec, prefix=""):
            return [TensorDecl(spec["name"], (int(spec["vocab_size"]), int(spec["dim"]))),
                    TensorDecl(spec["positions_name"], (int(spec["max_positions"]), int(spec["dim"])))]

        def load(self, store, prefix, device):
            self.table = store.get(self.spec["name"], torch.float32, device)
            self.places = store.get(self.spec["positions_name"], torch.float32, device)

        def forward(self, ids, ctx):
            return kernels.embed(self.table, ids) + self.places.index_select(0, ctx.positions.long())

    @dataclass(frozen=True)
    class ToyConfig:
        vocab_size: int
        architecture: str = "ToyDeviceStateForCausalLM"

        @classmethod
        def from_dict(cls, raw, where="config.json"):
            return cls(int(raw["vocab_size"]))

        def to_dict(self):
            return {"architectures": [self.architecture], "vocab_size": self.vocab_size}

    def toy_spec(cfg):
        norm = PartSpec("rmsnorm", dict(dim=H, eps=1e-5))
        ffn = PartSpec("gated_mlp", dict(hidden_size=H, intermediate_size=48, activation="silu"))
        rope = PartSpec("rope", dict(head_dim=D, rotary_dim=D, theta=10000.0, max_positions=POSITIONS))
        attn = PartSpec("attention", dict(hidden_size=H, num_heads=2, num_kv_heads=1, head_dim=D, qk_norm=False,
                                          window=None, position=rope, scale=0.25))
        norms = {"input_layernorm": norm, "post_attention_layernorm": norm}
        layers = (LayerSpec("model.layers.0", "prenorm", PartSpec("decayed_sum", dict(hidden_size=H, decay=DECAY)), ffn, norms),
                  LayerSpec("model.layers.1", "prenorm", attn, ffn, norms))
        return ModelSpec(
            architecture=cfg.architecture, vocab_size=cfg.vocab_size, hidden_size=H, max_positions=POSITIONS,
            embedding=PartSpec("embedding_with_positions", dict(name="wte.weight", positions_name="wpe.weight",
                                                                vocab_size=cfg.vocab_size, dim=H, max_positions=POSITIONS)),
            layers=layers, schedule=(ScheduleEntry(0), ScheduleEntry(1)),
            final_norm=PartSpec("rmsnorm", dict(dim=H, eps=1e-5, name="model.norm.weight")),
            head=PartSpec("lm_head", dict(name="lm_head.weight", tied=False, vocab_size=cfg.vocab_size, dim=H)))

    register_architecture("ToyDeviceStateForCausalLM", ModelFamily("toy_device_state", ToyConfig, toy_spec))


@pytest.fixture(scope="module")
def toy(tmp_path_factory):
    from xinfer_amd.engine import load_model
    from xinfer_amd.weights import write_random_model
    _register()
    d = write_random_model(str(tmp_path_factory.mktemp("toy_state") / "m"),
                           {"architectures": ["ToyDeviceStateForCausalLM"], "vocab_size": V}, seed=8, linear_std=0.15)
    model = load_model(d, "float32", DEV)
    W = plain.read_weights(d)
    cos, sin = plain.rope_tables(10000.0, D, POSITIONS)

    def logits(ids):
        """The same model written out plainly, a whole sequence at a time."""
        T = len(ids)
        x = W["wte.weight"][torch.tensor(ids)] + W["wpe.weight"][:T]
        h = plain.rms_norm(x, W["model.layers.0.input_layernorm.weight"], 1e-5)
        s, rows = torch.zeros(H), []
        for t in range(T):
            s = DECAY * s + h[t]
            rows.append(s)
        r = x + torch.stack(rows) @ W["model.layers.0.self_attn.mix.weight"].T
        x = r + plain.mlp_block(plain.rms_norm(r, W["model.layers.0.post_attention_layernorm.weight"], 1e-5), W, "model.layers.0.mlp")
        h = plain.rms_norm(x, W["model.layers.1.input_layernorm.weight"], 1e-5)
        pos = torch.arange(T)
        q = plain.apply_rope((h @ W["model.layers.1.self_attn.q_proj.weight"].T).reshape(T, 2, D), pos, cos, sin)
        k = plain.apply_rope((h @ W["model.layers.1.self_attn.k_proj.weight"].T).reshape(T, 1, D), pos, cos, sin)
        v = (h @ W["model.layers.1.self_attn.v_proj.weight"].T).reshape(T, 1, D)
        r = x + plain.attention(q, k, v, scale=0.25).reshape(T, 2 * D) @ W["model.layers.1.self_attn.o_proj.weight"].T
        x = r + plain.mlp_block(plain.rms_norm(r, W["model.layers.1.post_attention_layernorm.weight"], 1e-5), W, "model.layers.1.mlp")
        return plain.rms_norm(x, W["model.norm.weight"], 1e-5) @ W["lm_head.weight"].T

    return model, logits


def test_toy_device_state_and_position_embedding_under_every_cutting(toy):
    """Registered, written, loaded and stepped whole, in portions, mixed with few pages and with
    a tail of single tokens, without a change to the framework's files; the state slots are used
    again by later requests (two slots for five requests)."""
    from xinfer_amd.engine import ModelRunner
    model, toy_logits = toy
    assert model.graph_safe and set(model.state_needs) == {0} and set(model.kv_needs) == {1}
    rng = random.Random(21)
    reqs = {f"q{i}": harness.random_prompt(rng, n, V) for i, n in enumerate([23, 58, 4, 35, 91])}
    ref = {rid: toy_logits(t) for rid, t in reqs.items()}
    for what, steps in (("whole", harness.trace_whole(reqs)), ("mixed", harness.trace_mixed(reqs, 3, max_live=2)),
                        ("portions", harness.trace_portions(reqs)), ("tail", harness.trace_tail_one_by_one(reqs, tail=20))):
        runner = ModelRunner(model, page_size=8, num_pages=harness.tokens_needed(steps, 8) // 8, max_requests=2)
        harness.compare(harness.replay(runner, steps), ref, harness.TOL["float32"], f"toy device state {what}")


def test_a_recorded_step_advances_state_once(toy):
    """Four requests that start at different steps (one of them with a single token, inside a
    step of single tokens) decode together for a dozen steps.  With graphs recorded at the first
    sight of a batch size, every step that records and every replay gives the logits of the same
    steps launched kernel by kernel, bit for bit, and those of the plain model: the state is
    advanced once a step, in the recording step too."""
    from xinfer_amd.engine import ModelRunner
    model, toy_logits = toy
    rng = random.Random(22)
    toks = {rid: harness.random_prompt(rng, n, V) for rid, n in (("a", 30), ("b", 27), ("c", 22), ("d", 9))}
    fed = {rid: 0 for rid in toks}
    steps = []

    def step(parts, end=()):
        entries = []
        for rid, n in parts:
            entries.append({"id": rid, "tokens": toks[rid][fed[rid]:fed[rid] + n], "want": list(range(n))})
            fed[rid] += n
        steps.append({"step": len(steps), "entries": entries, "end": list(end)})

    step([("a", 9)])
    step([("a", 1)])                                     # one request alone: recorded
    step([("a", 1), ("b", 6)])                           # a portion beside a single token: launched
    for _ in range(2):
        step([("a", 1), ("b", 1)])                       # two: recorded, replayed
    step([("a", 1), ("b", 1), ("c", 5)])
    for _ in range(3):
        step([("a", 1), ("b", 1), ("c", 1)])             # three: recorded, replayed twice
    for _ in range(6):
        step([("a", 1), ("b", 1), ("c", 1), ("d", 1)])   # d starts with one token in a step of single tokens
    step([("a", 1), ("b", 1), ("c", 1)], end=["c"])
    for _ in range(3):
        step([("a", 1), ("b", 1), ("d", 1)])             # three again, other slots: the graph of three is replayed
    assert all(fed[rid] <= len(toks[rid]) for rid in toks)

    def run(**kw):
        runner = ModelRunner(model, page_size=8, num_pages=16, max_requests=4, **kw)
        return harness.replay(runner, steps), runner

    want, _ = run(use_graphs=False)
    got, runner = run(graph_after=1)
    assert {k[0] for k in runner._graphs} == {1, 2, 3, 4} and runner.graph_replays >= 8
    for key in sorted(want):
        assert torch.equal(want[key], got[key]), f"request {key[0]} position {key[1]} differs between graph and launches"
    ref = {rid: toy_logits(t[:fed[rid]]) for rid, t in toks.items()}
    harness.compare(got, ref, harness.TOL["float32"], "toy device state under graphs")
