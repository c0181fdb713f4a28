"""Weights by tensor name.

A `WeightStore` answers `get(name)` for every tensor of a model.  Two sources exist:
the safetensors files of a model folder, and seeded random values.  Parts declare the
tensors they need (`TensorDecl`), the model collects the declarations, and `check`
compares them with what the source holds before anything is loaded, so that a broken
checkpoint produces one error that lists every missing and mis-shaped tensor, and beside
them the tensors the model did not ask for (a misnamed tensor shows up as one of each);
the reference surfaces these one at a time as candle errors
(/root/reference/src/models/layers/mod.rs:170-194).  Tensors the model does not ask for
are no error by themselves: the reference reads by name and never looks at the rest (a
tied checkpoint that also stores lm_head.weight, an old export's rotary_emb.inv_freq;
/root/reference/src/models/qwen3.rs:267-287), so `check` returns their names and the
loader says once that it leaves them alone.

Storage policy: floating tensors are kept in bfloat16, except that a tensor stored in
32 bits stays in 32 bits; integer tensors become int32.  Parts ask for the compute
dtype they need (`get(name, dtype)`); norm weights are always used in float32
(/root/reference/src/models/qwen3.rs:83).
"""
from __future__ import annotations

import hashlib
import json
import os
from dataclasses import dataclass
from typing import Dict, Iterable, List, Optional, Sequence, Tuple

import torch

from .safetensors_io import SafetensorsFile


class WeightError(RuntimeError):
    """One error for everything that is wrong with a checkpoint: missing tensors and wrong
    shapes; the tensors nobody asked for are listed with them."""

    def __init__(self, where: str, missing: Sequence[str], unexpected: Sequence[str],
                 wrong_shape: Sequence[Tuple[str, Tuple[int, ...], Tuple[int, ...]]]):
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        lines = [f"weights in {where} do not match the model:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}):")
            lines += [f"    {n}" for n in self.missing]
        if self.unexpected:
            lines.append(f"  unexpected tensors, which the model does not use ({len(self.unexpected)}):")
            lines += [f"    {n}" for n in self.unexpected]
        if self.wrong_shape:
            lines.append(f"  wrong shapes ({len(self.wrong_shape)}):")
            lines += [f"    {n}: file has {list(got)}, model needs {list(want)}"
                      for n, got, want in self.wrong_shape]
        super().__init__("\n".join(lines))


@dataclass(frozen=True)
class TensorDecl:
    """A tensor a part needs.  `init` names how random weights fill it:
    "linear" ~ N(0, linear_std), "norm" ~ 1 + N(0, norm_std), "zeros"."""
    name: str
    shape: Tuple[int, ...]
    init: str = "linear"


def _storage_dtype(dt: torch.dtype) -> torch.dtype:
    if dt in (torch.float32,):
        return torch.float32
    if dt.is_floating_point:
        return torch.bfloat16
    if dt is torch.bool:
        return torch.bool
    return torch.int32


class WeightStore:
    """Common interface of the two sources."""

    where = "<weights>"

    def names(self) -> List[str]:
        raise NotImplementedError

    def shape(self, name: str) -> Tuple[int, ...]:
        raise NotImplementedError

    def _raw(self, name: str, device) -> torch.Tensor:
        raise NotImplementedError

    def has(self, name: str) -> bool:
        return name in set(self.names())

    def get(self, name: str, dtype: Optional[torch.dtype] = None, device="cpu") -> torch.Tensor:
        """The tensor under the storage policy, or converted to `dtype` if given."""
        t = self._raw(name, device)
        want = dtype if dtype is not None else _storage_dtype(t.dtype)
        return t.to(device=device, dtype=want)

    def check(self, decls: Iterable[TensorDecl]) -> List[str]:
        """Raises one `WeightError` if a declared tensor is missing or has another shape.
        Returns the names of the tensors that no declaration asks for."""
        decls = list(decls)
        have = set(self.names())
        want: Dict[str, Tuple[int, ...]] = {}
        for d in decls:
            want.setdefault(d.name, tuple(d.shape))
        missing = sorted(n for n in want if n not in have)
        unexpected = sorted(n for n in have if n not in want)
        wrong = sorted((n, self.shape(n), s) for n, s in want.items()
                       if n in have and tuple(self.shape(n)) != tuple(s))
        if missing or wrong:
            raise WeightError(self.where, missing, unexpected, wrong)
        return unexpected


class SafetensorsStore(WeightStore):
    """`model.safetensors.index.json` -> its shard files, else `model.safetensors`
    (/root/reference/src/utils/downloader.rs:170-177, src/utils/mod.rs:106-125)."""

    def __init__(self, model_dir: str):
        self.where = model_dir
        index = os.path.join(model_dir, "model.safetensors.index.json")
        single = os.path.join(model_dir, "model.safetensors")
        if os.path.isfile(index):
            with open(index, "r", encoding="utf-8") as f:
                files = sorted(set(json.load(f)["weight_map"].values()))
        elif os.path.isfile(single):
            files = ["model.safetensors"]
        else:
            raise FileNotFoundError(f"No weight files found in {model_dir!r} "
                                    "(model.safetensors or model.safetensors.index.json)")
        self._files = [SafetensorsFile(os.path.join(model_dir, f)) for f in files]
        self._where_is: Dict[str, SafetensorsFile] = {}
        for sf in self._files:
            for n in sf.names():
                if n in self._where_is:
                    raise ValueError(f"tensor {n!r} appears in two weight files of {model_dir!r}")
                self._where_is[n] = sf

    def names(self) -> List[str]:
        return list(self._where_is)

    def has(self, name: str) -> bool:
        return name in self._where_is

    def shape(self, name: str) -> Tuple[int, ...]:
        return self._where_is[name].shape(name)

    def _raw(self, name: str, device) -> torch.Tensor:
        return self._where_is[name].tensor(name)

    def close(self) -> None:
        for sf in self._files:
            sf.close()


class RandomStore(WeightStore):
    """Seeded random weights: element i of a tensor is a normal value made from (seed, the
    tensor's name, i) alone (`counter_normal`), so a tensor's values do not depend on which
    others exist, on order, or on the device they are made on: the GPU's kernel and the CPU's
    numpy twin give the same bits.  Values are rounded to `dtype` (bfloat16 unless told
    otherwise), as a checkpoint's are."""

    def __init__(self, decls: Iterable[TensorDecl], seed: int, linear_std: float = 0.02,
                 norm_std: float = 0.1, dtype: torch.dtype = torch.bfloat16):
        self.where = f"<random weights, seed {seed}>"
        self._decls: Dict[str, TensorDecl] = {}
        for d in decls:
            self._decls.setdefault(d.name, d)
        self.seed = int(seed)
        self.linear_std = float(linear_std)
        self.norm_std = float(norm_std)
        self.dtype = dtype

    def names(self) -> List[str]:
        return list(self._decls)

    def has(self, name: str) -> bool:
        return name in self._decls

    def shape(self, name: str) -> Tuple[int, ...]:
        return tuple(self._decls[name].shape)

    def _tensor_key(self, name: str) -> int:
        h = hashlib.sha256(f"{self.seed}:{name}".encode("utf-8")).digest()
        return int.from_bytes(h[:8], "little")

    def _raw(self, name: str, device) -> torch.Tensor:
        d = self._decls[name]
        dev = torch.device(device)
        if d.init == "zeros":
            return torch.zeros(d.shape, dtype=self.dtype, device=dev)
        if d.init == "norm":
            scale, shift = self.norm_std, 1.0
        elif d.init == "linear":
            scale, shift = self.linear_std, 0.0
        else:
            raise ValueError(f"tensor {name!r}: unknown init {d.init!r}")
        key = self._tensor_key(name)
        t = torch.empty(d.shape, dtype=self.dtype, device=dev)
        flat = t.view(-1)
        n = flat.numel()
        if dev.type == "cuda":
            from .. import kernels
            with torch.cuda.device(dev):
                if self.dtype in (torch.float32, torch.bfloat16):
                    kernels.counter_normal_(flat, key, scale, shift)
                else:                # in pieces, so that a large table needs no float32 twin
                    step = 1 << 26
                    for b in range(0, n, step):
                        piece = torch.empty((min(step, n - b),), dtype=torch.float32, device=dev)
                        flat[b:b + piece.numel()] = kernels.counter_normal_(piece, key, scale, shift, first=b).to(self.dtype)
            return t
        from .counter_normal import counter_normal
        step = 1 << 20

        def piece(b: int) -> None:
            m = min(step, n - b)
            flat[b:b + m] = torch.from_numpy(counter_normal(key, b, m, scale, shift)).to(self.dtype)

        starts = range(0, n, step)
        if len(starts) > 1:          # numpy works outside the interpreter's lock
            from concurrent.futures import ThreadPoolExecutor
            with ThreadPoolExecutor(min(8, len(starts))) as ex:
                list(ex.map(piece, starts))
        else:
            for b in starts:
                piece(b)
        return t
