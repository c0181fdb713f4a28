"""Choice of the sampling strategy per request and the draw itself.

Strategies and their precedence follow the reference: temperature below 1e-7 or absent
means greedy (/root/reference/src/utils/logits_processor.rs:48-65); a request's own
parameters come before the model's generation defaults, and with neither the default is
top-k 32, top-p 0.95, temperature 0.7 (/root/reference/src/core/runner.rs:1803-1854).
The reference picks one strategy per batch from its first sequence and draws from one
shared generator; here every request has its own strategy and its own stream of random
numbers (seed, request, number of tokens drawn so far), so a request's tokens do not
depend on what it was batched with.  Frequency and presence penalties count what the
reference counts (`penalty_context`, `penalties_apply`): the last 128 sampled tokens once
more than 128 were sampled, never the prompt, and a penalty of exactly 1.0 counts as off.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Sequence

import numpy as np
import torch

from .. import kernels
from ..config.engine_config import GenerationConfig, SamplingParams

TOPK_FAST = 64             # largest top-k of the two-stage selection (`sampling_topk.hip`)
PENALTY_CONTEXT = 128      # tokens that penalties look at (runner.rs:1887-1912)
_MASK = (1 << 64) - 1


@dataclass(frozen=True)
class Strategy:
    temperature: float = 0.0    # 0: greedy
    top_k: int = 0              # 0: no limit
    top_p: float = 1.0          # 1: no limit
    frequency_penalty: float = 0.0
    presence_penalty: float = 0.0

    @property
    def greedy(self) -> bool:
        return self.temperature < 1e-7


def get_strategy(temperature: Optional[float], top_k: Optional[int], top_p: Optional[float]) -> Strategy:
    """LogitsProcessor::get_strategy (logits_processor.rs:48-65)."""
    if temperature is None or temperature < 1e-7:
        return Strategy()
    k = int(top_k) if (top_k is not None and top_k > 0) else 0
    p = float(top_p) if top_p is not None else 1.0
    return Strategy(float(temperature), k, p)


def resolve_strategy(params: SamplingParams, defaults: Optional[GenerationConfig]) -> Strategy:
    """Precedence of runner.rs:1803-1854."""
    freq = params.frequency_penalty if params.frequency_penalty is not None else \
        (defaults.frequency_penalty if defaults else None)
    pres = params.presence_penalty if params.presence_penalty is not None else \
        (defaults.presence_penalty if defaults else None)
    has_user = (params.temperature is not None or (params.top_k is not None and params.top_k > 0)
                or (params.top_p is not None and 0.0 < params.top_p < 1.0))
    if params.temperature is not None and params.temperature == 0.0:
        s = Strategy()
    elif has_user:
        s = get_strategy(params.temperature, params.top_k, params.top_p)
    elif defaults is not None and defaults.temperature is not None and (
            defaults.top_k is not None or defaults.top_p is not None):
        s = get_strategy(defaults.temperature, defaults.top_k, defaults.top_p)
    else:
        s = Strategy(0.7, 32, 0.95)
    return Strategy(s.temperature, s.top_k, s.top_p, float(freq or 0.0), float(pres or 0.0))


def penalty_context(tokens: Sequence[int], prompt_len: int) -> List[int]:
    """The tokens that frequency and presence penalties count for a request whose prompt and
    generated tokens are `tokens`: the last PENALTY_CONTEXT of the tokens sampled so far (the
    prompt is not among them: the reference's list holds what was sampled, runner.rs:1950-1962),
    and none until more than PENALTY_CONTEXT have been sampled (runner.rs:1892-1897), so the
    first token that penalties touch is the 130th generated one."""
    generated = len(tokens) - prompt_len
    if generated <= PENALTY_CONTEXT:
        return []
    return list(tokens[len(tokens) - PENALTY_CONTEXT:])


def penalties_apply(strategy: Strategy, context: Sequence[int]) -> bool:
    """Whether a row's penalties are applied (logits_processor.rs:399-401): more than one token
    to count, and one of the two penalties neither 0 nor exactly 1 (the reference takes 1.0 for
    "off" too); both values are then subtracted as they are."""
    on = lambda v: v != 0.0 and v != 1.0
    return len(context) > 1 and (on(strategy.frequency_penalty) or on(strategy.presence_penalty))


def uniform(seed: int, request: int, draw: int) -> float:
    """The draw-th uniform number in [0, 1) of a request's stream: splitmix64 of the three
    counters, 24 bits kept so that the float32 value is exact."""
    x = (seed * 0x9E3779B97F4A7C15 + request * 0xBF58476D1CE4E5B9 + draw * 0x94D049BB133111EB + 0x2545F4914F6CDD1D) & _MASK
    for _ in range(2):
        x = (x + 0x9E3779B97F4A7C15) & _MASK
        z = x
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
        x = z ^ (z >> 31)
    return (x >> 40) / float(1 << 24)


class Sampler:
    """Draws one token per row of float32 logits on the GPU."""

    def __init__(self, device):
        self.device = torch.device(device)
        lib = kernels.lib()
        self._lib = lib
        self._pin: Optional[torch.Tensor] = None
        self._pin_free = None

    def argmax(self, logits: torch.Tensor) -> torch.Tensor:
        kernels._dev(logits)
        kernels._want(logits, torch.float32, "argmax: logits")
        if logits.dim() != 2:
            raise kernels.KernelError("argmax: logits must be [rows, vocab]")
        rows, V = logits.shape
        out = torch.empty((rows,), dtype=torch.int32, device=logits.device)
        chunks = int(self._lib.xi_argmax_chunks(V))
        pval = pidx = None
        if chunks > 1:
            pval = torch.empty((rows, chunks), dtype=torch.float32, device=logits.device)
            pidx = torch.empty((rows, chunks), dtype=torch.int32, device=logits.device)
        kernels._ok(self._lib.xi_argmax(kernels._p(logits), rows, V, kernels._p(out), kernels._p(pval),
                                        kernels._p(pidx), kernels._stream()))
        return out

    def sample(self, logits: torch.Tensor, strategies: Sequence[Strategy], uniforms: Sequence[float],
               recent: Optional[Sequence[Sequence[int]]] = None) -> List[int]:
        """logits float32 [R, V] (changed in place when penalties apply); one strategy and
        one uniform number per row; `recent[r]` = the tokens the row's penalties count
        (`penalty_context`).  Returns R token ids."""
        return self.sample_device(logits, strategies, uniforms, recent).tolist()

    def _params(self, rows: Sequence[Sequence[float]]) -> torch.Tensor:
        """Per-row numbers as a float32 tensor [len(rows), R] on the device, by way of pinned memory:
        a copy from ordinary memory makes the host wait for the GPU's earlier work."""
        n, R = len(rows), len(rows[0])
        if self._pin is None or self._pin.numel() < n * R:
            self._pin = torch.empty((max(1024, n * R),), dtype=torch.float32, pin_memory=True)
        if self._pin_free is not None:
            self._pin_free.synchronize()         # the copy before has left the buffer
        host = self._pin[:n * R].view(n, R)
        host.copy_(torch.tensor(rows, dtype=torch.float32))
        out = torch.empty((n, R), dtype=torch.float32, device=self.device)
        out.copy_(host, non_blocking=True)
        self._pin_free = torch.cuda.Event()
        self._pin_free.record()
        return out

    def sample_device(self, logits: torch.Tensor, strategies: Sequence[Strategy], uniforms: Sequence[float],
                      recent: Optional[Sequence[Sequence[int]]] = None) -> torch.Tensor:
        """`sample` without the copy to the host: the R token ids as an int32 tensor on the device;
        nothing here waits for the GPU (unless penalties apply)."""
        kernels._dev(logits)
        kernels._want(logits, torch.float32, "sample: logits")
        R, V = logits.shape
        if R != len(strategies) or R != len(uniforms):
            raise kernels.KernelError("sample: one strategy and one uniform number per row are needed")
        dev = logits.device
        if R == 0:
            return torch.empty((0,), dtype=torch.int32, device=dev)
        if recent is not None and any(penalties_apply(s, rc) for s, rc in zip(strategies, recent)):
            n = PENALTY_CONTEXT
            rec = np.full((R, n), -1, dtype=np.int32)
            fr = np.zeros(R, dtype=np.float32)
            pr = np.zeros(R, dtype=np.float32)
            for r, (s, rc) in enumerate(zip(strategies, recent)):
                rc = list(rc)[-n:]
                if penalties_apply(s, rc):
                    rec[r, :len(rc)] = rc
                    fr[r], pr[r] = s.frequency_penalty, s.presence_penalty
            rec_d, fr_d, pr_d = (torch.from_numpy(a).to(dev) for a in (rec, fr, pr))
            kernels._ok(self._lib.xi_apply_penalties(kernels._p(logits), R, V, kernels._p(rec_d), n,
                                                     kernels._p(fr_d), kernels._p(pr_d), kernels._stream()))
        if all(s.greedy for s in strategies):
            return self.argmax(logits)
        chunks = int(self._lib.xi_sample_topk_chunks(V))
        if chunks > 0 and all(s.greedy or 1 <= s.top_k <= TOPK_FAST for s in strategies):
            # a small top-k everywhere (the default strategy has 32): the k most probable of a row
            # are found by many workgroups, the rest is about k numbers
            par = self._params([[s.temperature for s in strategies], [float(s.top_k) for s in strategies],
                                [s.top_p for s in strategies], list(uniforms)])
            cand_v = torch.empty((R, chunks, TOPK_FAST), dtype=torch.float32, device=dev)
            cand_i = torch.empty((R, chunks, TOPK_FAST), dtype=torch.int32, device=dev)
            out = torch.empty((R,), dtype=torch.int32, device=dev)
            kernels._ok(self._lib.xi_sample_topk(kernels._p(logits), R, V, kernels._p(par), kernels._p(cand_v),
                                                 kernels._p(cand_i), kernels._p(out), kernels._stream()))
            return out
        t, kf, p, u = self._params([[s.temperature for s in strategies], [float(s.top_k) for s in strategies],
                                    [s.top_p for s in strategies], list(uniforms)])
        k = kf.to(torch.int32)              # (a row's top_k is far below 2^24: exact as float32)
        probs = torch.empty_like(logits)
        out = torch.empty((R,), dtype=torch.int32, device=dev)
        kernels._ok(self._lib.xi_sample(kernels._p(logits), R, V, kernels._p(t), kernels._p(k), kernels._p(p),
                                        kernels._p(u), kernels._p(probs), kernels._p(out), kernels._stream()))
        return out
