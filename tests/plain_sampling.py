"""Plain sampling on the CPU, from the reference's formulas
(/root/reference/src/utils/logits_processor.rs): probabilities are softmax(logits / T) in
float32 (:305-320); top-k keeps the k most probable (:113-141); top-p keeps, in descending
order, each token whose preceding cumulative mass is below p (:82-111); top-k then top-p
applies the cutoff to the renormalised top-k set (:143-200); penalties subtract
count * frequency + [count > 0] * presence (:358-378).  Ties are ordered by token id.  The
draw walks the kept tokens in token order with a given uniform number."""
from typing import Sequence

import torch


def kept_probabilities(logits: torch.Tensor, temperature: float, top_k: int = 0, top_p: float = 1.0) -> torch.Tensor:
    """Unnormalised probabilities with the tokens outside the kept set at zero."""
    p = torch.softmax(logits.double() / temperature, dim=-1)
    V = p.numel()
    order = sorted(range(V), key=lambda i: (-float(p[i]), i))
    keep = order
    if 0 < top_k < V:
        keep = order[:top_k]
    if 0.0 < top_p < 1.0:
        mass = float(sum(p[i] for i in keep))
        cum, cut = 0.0, []
        for i in keep:
            if cum >= top_p * mass:
                break
            cum += float(p[i])
            cut.append(i)
        keep = cut
    out = torch.zeros_like(p)
    idx = torch.tensor(keep)
    out[idx] = p[idx]
    return out


def draw(kept: torch.Tensor, u: float) -> int:
    goal = u * float(kept.sum())
    cum = torch.cumsum(kept, 0)
    nz = torch.nonzero((cum > goal) & (kept > 0))
    return int(nz[0]) if len(nz) else int(torch.nonzero(kept > 0)[-1])


def apply_penalties(logits: torch.Tensor, context: Sequence[int], frequency: float, presence: float) -> torch.Tensor:
    out = logits.clone()
    counts = {}
    for t in context:
        counts[t] = counts.get(t, 0) + 1
    for t, c in counts.items():
        out[t] = out[t] - c * frequency - presence
    return out
