"""Rotary position embedding (half-split rotation), reference interface
nanovllm/layers/rotary_embedding.py:92-205; kernel nvh_rope in csrc/elementwise.hip.

The cos|sin table is built on the HOST in fp32 with the reference's formula and then
moved to the device, so every rank and the CPU oracle rotate with bit-identical tables.
"""
from functools import lru_cache

import torch
from torch import nn

from .. import ops


class RotaryEmbedding(nn.Module):
    def __init__(self, head_size: int, rotary_dim: int, max_position_embeddings: int, base: float) -> None:
        super().__init__()
        assert rotary_dim == head_size
        self.head_size = head_size
        cpu = torch.device("cpu")
        inv_freq = 1.0 / (base ** (torch.arange(0, rotary_dim, 2, dtype=torch.float, device=cpu) / rotary_dim))
        t = torch.arange(max_position_embeddings, dtype=torch.float, device=cpu)
        freqs = torch.outer(t, inv_freq)
        cache = torch.cat((freqs.cos(), freqs.sin()), dim=-1).unsqueeze_(1)      # [max_pos, 1, D]
        self.register_buffer("cos_sin_cache", cache.to(torch.empty(0).device), persistent=False)

    def table2d(self) -> torch.Tensor:
        return self.cos_sin_cache.view(self.cos_sin_cache.shape[0], self.head_size)

    def forward(self, positions: torch.Tensor, query: torch.Tensor, key: torch.Tensor):
        """Rotates query [T,Hq,D] and key [T,Hkv,D] IN PLACE and returns them."""
        ops.rope_(positions, query, key, self.table2d())
        return query, key


@lru_cache(1)
def _cached_rope(head_size: int, rotary_dim: int, max_position: int, base: float):
    return RotaryEmbedding(head_size, rotary_dim, max_position, base)


def get_rope(head_size: int, rotary_dim: int, max_position: int, base: float, rope_scaling: dict | None = None):
    """One shared module per process (all layers use the same table)."""
    if rope_scaling is not None:
        kind = rope_scaling.get("rope_type", "default")
        assert kind == "default", f"rope_type '{kind}' is not supported"
    return _cached_rope(head_size, rotary_dim, max_position, float(base))


def rotary_frequencies(dims: int, base: float, yarn: dict | None = None) -> tuple[torch.Tensor, float]:
    """(fp32 frequencies of the dims/2 rotation pairs, factor on cos and sin) for kernels that form the angle
    position * frequency themselves (nvh_attn_rotary_prep), so no table bounds the position.

    Without `yarn`: base^(-2i/dims) and 1.  With yarn = {factor, original, fast, slow} (YaRN: "Efficient Context Window
    Extension of Large Language Models", Peng et al.): a pair that turns more than `fast` times over the `original`
    context keeps its frequency, one that turns fewer than `slow` times is divided by `factor`, pairs in between blend
    linearly in the pair index; cos and sin are scaled by 0.1 ln(factor) + 1.  Computed in float64 on the host."""
    import math
    half = dims // 2
    freq = [base ** (-2.0 * i / dims) for i in range(half)]
    if not yarn:
        return torch.tensor(freq, dtype=torch.float64).float(), 1.0
    factor, original = float(yarn["factor"]), float(yarn["original"])

    def pair_index(turns: float) -> float:         # the (fractional) pair that makes `turns` turns over the original context
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(pair_index(float(yarn["fast"]))), 0)
    hi = min(math.ceil(pair_index(float(yarn["slow"]))), dims - 1)
    out = []
    for i, f in enumerate(freq):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f / factor * ramp + f * (1.0 - ramp))
    return torch.tensor(out, dtype=torch.float64).float(), 0.1 * math.log(factor) + 1.0


def banded_frequencies(dims: int, base: float, scaling: dict | None = None) -> torch.Tensor:
    """fp32 frequencies of the dims/2 rotation pairs, f_i = base^(-2i/dims), under a context-extension rule (float64 on the host):

      scaling None                              the plain frequencies;
      {factor}                                  position interpolation: every f_i / factor;
      {factor, low, high, original}             the rule of Llama 3.1 by wavelength l = 2 pi / f: pairs with l < original / high keep
                                                f, pairs with l > original / low take f / factor, and in between
                                                s = (original / l - low) / (high - low) blends them, (1 - s) f / factor + s f."""
    import math
    freq = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    if scaling:
        factor = float(scaling["factor"])
        if "original" in scaling:
            low, high, original = float(scaling["low"]), float(scaling["high"]), float(scaling["original"])
            out = []
            for f in freq:
                wavelength = 2.0 * math.pi / f
                if wavelength < original / high:
                    out.append(f)
                elif wavelength > original / low:
                    out.append(f / factor)
                else:
                    s = (original / wavelength - low) / (high - low)
                    out.append((1.0 - s) * f / factor + s * f)
            freq = out
        else:
            freq = [f / factor for f in freq]
    return torch.tensor(freq, dtype=torch.float64).float()
