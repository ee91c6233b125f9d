"""Weights by tensor name: what a model asks for is checked against what a source holds, once.

The reference loads every tensor by its canonical name and checks each shape a kernel relies on against
the config (model/ModelWeights.java:28-84, model/DecoderLayer.java:20-44, model/AttnWeights.java:33-64,
model/MlpWeights.java:23-39). Here every part declares its tensors as ``WeightSpec``s; ``check`` compares
the whole list with the source and raises ONE error that lists missing tensors, unexpected tensors and
wrong shapes; ``fetch`` then brings each tensor to the device in the storage dtype of the run.

Storage rule: floating tensors stored in 16 bits are kept in bfloat16 in a bfloat16 run; a tensor stored
in 32 bits stays 32-bit; integer tables become int32. A float32 run holds every floating tensor in float32
(an exact widening).
"""
from __future__ import annotations

import zlib
from dataclasses import dataclass
from typing import Dict, List, Sequence, Tuple

import torch


class WeightError(ValueError):
    """Raised once per load with everything that is wrong."""

    def __init__(self, missing, unexpected, wrong_shape, where: str = ""):
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        lines = [f"weights do not match the configuration{(' (' + where + ')') if where else ''}:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(f"  wrong shapes ({len(self.wrong_shape)}): " + "; ".join(
                f"{n} is {list(got)}, expected {list(exp)}" for n, got, exp in self.wrong_shape))
        super().__init__("\n".join(lines))


@dataclass(frozen=True)
class WeightSpec:
    """One tensor a part needs. ``init`` tells the random-weights mode how to fill it:
    "matrix" N(0, std), "gain" 1 + N(0, gain_std), "bias" N(0, std), "zeros"."""

    name: str
    shape: Tuple[int, ...]
    init: str = "matrix"
    optional: bool = False


def check(specs: Sequence[WeightSpec], source, where: str = "") -> None:
    have = set(source.names())
    wanted = {s.name for s in specs}
    missing = [s.name for s in specs if not s.optional and s.name not in have]
    unexpected = sorted(have - wanted)
    wrong = []
    for s in specs:
        if s.name in have and tuple(source.shape(s.name)) != tuple(s.shape):
            wrong.append((s.name, tuple(source.shape(s.name)), tuple(s.shape)))
    if missing or unexpected or wrong:
        raise WeightError(missing, unexpected, wrong, where)


def storage_dtype(stored: torch.dtype, run_dtype: torch.dtype) -> torch.dtype:
    if not stored.is_floating_point:
        return torch.int32
    if run_dtype == torch.float32:
        return torch.float32
    if stored in (torch.float32, torch.float64):
        return torch.float32
    return torch.bfloat16


def fetch(source, name: str, run_dtype: torch.dtype, device) -> torch.Tensor:
    t = source.get(name)
    want = storage_dtype(t.dtype, run_dtype)
    if t.device != torch.device(device):
        t = t.to(device=device, non_blocking=False)
    if t.dtype != want:
        t = t.to(want)
    return t.contiguous()


class TensorSource:
    """Tensors already in memory, by name, as a weight source (a model changed by hand, another loader's output)."""

    def __init__(self, tensors: Dict[str, torch.Tensor]):
        self.tensors = dict(tensors)

    def names(self) -> List[str]:
        return list(self.tensors)

    def shape(self, name: str) -> Tuple[int, ...]:
        return tuple(self.tensors[name].shape)

    def dtype(self, name: str) -> torch.dtype:
        return self.tensors[name].dtype

    def get(self, name: str) -> torch.Tensor:
        return self.tensors[name]


class RandomSource:
    """A source that makes each tensor from (seed, tensor name): the random-weights mode.

    Matrices, embeddings and biases are N(0, std); gains are 1 + N(0, gain_std) (exactly 1 when gain_std is
    0). Values are rounded to ``dtype`` so a written file and an in-memory source hold the same model. The
    generator runs on ``device``; a file written for tests uses the CPU generator.
    """

    def __init__(self, specs: Sequence[WeightSpec], seed: int, std: float = 0.02, gain_std: float = 0.1,
                 dtype: torch.dtype = torch.bfloat16, device="cpu"):
        self.specs: Dict[str, WeightSpec] = {s.name: s for s in specs if not s.optional}
        self.seed = int(seed)
        self.std = std
        self.gain_std = gain_std
        self._dtype = dtype
        self.device = torch.device(device)

    def names(self) -> List[str]:
        return list(self.specs)

    def shape(self, name: str) -> Tuple[int, ...]:
        return self.specs[name].shape

    def dtype(self, name: str) -> torch.dtype:
        return self._dtype

    def get(self, name: str) -> torch.Tensor:
        s = self.specs[name]
        g = torch.Generator(device=self.device)
        g.manual_seed((self.seed * 1000003 + zlib.crc32(name.encode("utf-8"))) % (2**63 - 1))
        if s.init == "zeros":
            return torch.zeros(s.shape, dtype=self._dtype, device=self.device)
        if s.init == "gain":
            if self.gain_std == 0:
                return torch.ones(s.shape, dtype=self._dtype, device=self.device)
            t = torch.randn(s.shape, generator=g, dtype=torch.float32, device=self.device) * self.gain_std + 1.0
        else:
            t = torch.randn(s.shape, generator=g, dtype=torch.float32, device=self.device) * self.std
        return t.to(self._dtype)
