"""Position encodings.  "rope": inv_freq[j] = 1 / theta^(2j / rotary_dim) built in
float32 exactly as the reference builds it (src/wllm/models/llama.py:52-56); the
angle position * inv_freq[j] and its sine and cosine are computed in float32
inside the rotation kernel (llama.py:58-62), and element j is paired with
j + rotary_dim/2 (llama.py:47-49,65-71).  The table stays float32 in every
mode.  Two options beyond that form: `pairing="interleaved"` pairs element 2j with 2j + 1, and
`scaling_factor` divides every frequency (linear scaling of positions); with either, the table
is worked out in float64 and rounded once.  `rotary_dim` may be less than the head: the rest of
a head passes unchanged.  `ramp` interpolates each pair's frequency between its plain value and that
value divided by a factor, by how many turns the pair makes within a given number of positions; and
`magnitude` (read by the rotation kernels as a factor of sine and cosine) scales what turns.
"none": no rotation."""
from __future__ import annotations

import math

import torch

from wllm_amd.parts.registry import register_position
from wllm_amd.parts.specs import PositionSpec


@register_position("rope")
class RotaryPosition:
    def __init__(self, spec: PositionSpec):
        if spec.pairing not in ("half", "interleaved"):
            raise ValueError(f"rope pairing {spec.pairing!r} is not implemented; 'half' or 'interleaved'")
        if not spec.scaling_factor > 0.0:
            raise ValueError(f"scaling_factor must be positive, got {spec.scaling_factor}")
        if spec.rotary_dim <= 0 or spec.rotary_dim % 2:
            raise ValueError(f"rotary_dim must be positive and even, got {spec.rotary_dim}")
        if spec.ramp is not None:
            factor, original, fast, slow = spec.ramp
            if not (factor > 0 and original > 0 and fast > 0 and slow > 0 and spec.theta > 1.0):
                raise ValueError(f"ramp (factor, original, fast, slow) must be positive and theta above 1, got {spec.ramp}")
        self.spec = spec
        self.inv_freq = None

    @property
    def magnitude(self) -> float:
        return float(self.spec.magnitude)

    def prepare(self, device) -> None:
        d = self.spec.rotary_dim
        if self.spec.ramp is not None:
            factor, original, fast, slow = (float(v) for v in self.spec.ramp)
            exact = 1.0 / (float(self.spec.theta) ** (torch.arange(0, d, 2, dtype=torch.float64) / d))
            exact = exact / self.spec.scaling_factor

            def pair_of(turns: float) -> float:
                return d * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(float(self.spec.theta)))

            lo = max(math.floor(pair_of(fast)), 0)
            hi = min(math.ceil(pair_of(slow)), d - 1)
            ramp = torch.clamp((torch.arange(d // 2, dtype=torch.float64) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
            inv = (exact / factor * ramp + exact * (1.0 - ramp)).to(torch.float32)
        elif self.spec.pairing == "half" and self.spec.scaling_factor == 1.0:
            inv = 1.0 / (self.spec.theta ** (torch.arange(0, d, 2, dtype=torch.float32) / d))
        else:
            exact = 1.0 / (float(self.spec.theta) ** (torch.arange(0, d, 2, dtype=torch.float64) / d))
            inv = (exact / self.spec.scaling_factor).to(torch.float32)
        self.inv_freq = inv.to(device)

    @property
    def interleaved(self) -> bool:
        return self.spec.pairing == "interleaved"


@register_position("none")
class NoPosition:
    def __init__(self, spec: PositionSpec):
        self.spec = spec
        self.inv_freq = None

    def prepare(self, device) -> None:
        pass
