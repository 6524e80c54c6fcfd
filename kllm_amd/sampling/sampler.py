"""Choosing the next token: greedy and temperature sampling.

The reference samples greedily only, on the host: the index of the largest
logit, the first one on ties (engine/engine.go:216-224); temperature is
described but not built (docs/theory/02-autoregressive-decoding.md:122-123).
Here both run on the device.  With temperature T > 0 the token is drawn from
softmax(logits / T) by inverting the cumulative distribution at a uniform
number; that number depends only on (the request's seed, how many tokens the
request has generated), never on what else is in the batch.  The logits
themselves equal those of the request alone up to rounding only (which kernel
runs, and how it cuts its sums, follows the step's size): a request samples the
same tokens alone and in any batch except where two candidates lie within that
rounding of each other, a last bit in float32, about a hundredth in bfloat16.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import List, Sequence

_MASK = (1 << 64) - 1


def _splitmix64(x: int) -> int:
    x = (x + 0x9E3779B97F4A7C15) & _MASK
    z = x
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return z ^ (z >> 31)


def uniform(seed: int, index: int) -> float:
    """A number in [0, 1) with 24 random bits (exact in float32), a pure
    function of (seed, index)."""
    z = _splitmix64(_splitmix64(seed & _MASK) ^ ((index * 0xD1342543DE82EF95) & _MASK))
    return (z >> 40) / float(1 << 24)


@dataclass(frozen=True)
class SamplingParams:
    temperature: float = 0.0   # 0: greedy
    seed: int = 0

    def uniform_for(self, generated_index: int) -> float:
        return uniform(self.seed, generated_index)


def sample_host(logits_rows, temperatures: Sequence[float], uniforms: Sequence[float]) -> List[int]:
    """The same choice on the host, for rows given as sequences of floats:
    used where no device is involved (tests of the scheduler with a stand-in
    engine)."""
    import math
    out = []
    for row, t, u in zip(logits_rows, temperatures, uniforms):
        row = [float(v) for v in row]
        best = 0
        for i in range(1, len(row)):
            if row[i] > row[best]:
                best = i
        if not t > 0:
            out.append(best)
            continue
        mx = row[best]
        e = [math.exp((v - mx) / t) for v in row]
        target = u * sum(e)
        c, idx = 0.0, len(row) - 1
        for i, v in enumerate(e):
            c += v
            if target < c:
                idx = i
                break
        out.append(idx)
    return out


class DeviceSampler:
    """Samples on the GPU with the sampling kernel; returns host ints."""

    def __init__(self, device):
        self.device = device

    def sample(self, logits, temperatures: Sequence[float], uniforms: Sequence[float]) -> List[int]:
        import torch
        from .. import kernels as K
        rows = logits.shape[0]
        out = torch.empty(rows, dtype=torch.int32, device=self.device)
        if any(t > 0 for t in temperatures):
            tu = torch.tensor([list(map(float, temperatures)), list(map(float, uniforms))],
                              dtype=torch.float32).to(self.device)
            K.sample(out, logits, tu[0].contiguous(), tu[1].contiguous())
        else:
            K.sample(out, logits)
        return out.tolist()
