"""Sokipel: a decoder-only stack over an fp32 residual stream whose sublayers read the stream itself and whose RESULTS are normed, with
three kinds of sequence mixers (chunked softmax attention with sinks, the gated delta rule, both side by side), a short causal
convolution of the stream in front of every mixer, and mixture-of-experts feed-forwards whose routing weight scales the expert's input.

    x = s_e * embed[token]                                 (s_e: the embedding scale)
    for every layer:
        h = x + conv(x)                                    (per column over time, `canon.taps` wide; layers.recurrent.StreamConv)
        x = x + m * g1 * unit(mixer(h))                    (unit(y) = y / sqrt(mean(y^2) + eps); g1, g2: ONE number each; m: residual_mult)
        x = x + m * g2 * unit(ff(x))                       (layers without a feed-forward skip this; the feed-forward reads x without the convolution)
    logits = cap * tanh(head(g_f * unit(x)) / cap)

Mixers (sizes and constants per layer from config.json; all softmax attention carries a learned sink logit per head):
  attention   q, k, v without biases; RMS norm over the whole q and the whole k projection; rotary in interleaved pairs with the
              wavelength-banded frequency rule of Llama 3.1; a query sees the earlier tokens of its own block of `mask.size` positions
  delta       layers.recurrent.GatedDeltaRule: short convolutions and silu on q, k, v, unit q and k, one decay and one write strength
              per head, per-head RMS read-out with a shared weight row, silu gate
  parallel    left_scale * left + right_scale * right over the one input: left = causal attention with q/k/v biases, an RMS norm per head
              (one weight row shared by the heads), rotary in halves with interpolated positions, and a sigmoid output gate per head;
              right = the gated delta rule
Feed-forward: layers.moe.SparseMoE with sigmoid scores (the `top` best, weights not renormalised, applied to the expert's input) and the
capped gated unit g = min(gate x, limit), u = clamp(up x, +-limit), y = g sigmoid(1.702 g) (u + 1).

32-bit whatever the activation type: positions and angles, the stream, its convolution and its sums, every norm, attention scores and
weights, router logits and scores, every operand of the recurrence (convolution sums, unit vectors, decays, write strengths, the state,
the read-out norm), the capped unit, the softcap.  Projections run in the model's dtype (bf16, or fp32 for a model served in full precision).

config.json keys: architecture, vocab, width, embedding.scale, residual_mult, logit_softcap, norm.eps, canon {taps} | null, layers[] of
{type, mixer {...}, mlp {kind: moe, expert {ff, limit}, router {experts, top}} | null}.  attention mixer: heads, kv_heads, dim, vdim,
scale, rot {base, dims, scaling {factor[, low, high, original]} | null} | null, mask {size} | null; delta: heads, kv_heads, dim, vdim,
conv; parallel: left {attention keys}, right {delta keys}, left_scale, right_scale.  Tensors: embed, head, final.norm, l<i>.norm1|norm2,
l<i>.canon1, l<i>.mix.*, l<i>.mlp.e<n>.gate|up|down, l<i>.mlp.router.
"""
from __future__ import annotations

import re
import zlib

import torch
from torch import nn

from .. import ops
from ..layers.attention import GatedValueRotaryAttention
from ..layers.layernorm import StreamNorm, SublayerOutputNorm
from ..layers.linear import MergedLinear
from ..layers.moe import SparseMoE
from ..layers.recurrent import GatedDeltaRule, StreamConv
from ..layers.rotary_embedding import banded_frequencies
from .lamutar import _get


class SokipelAttention(nn.Module):
    """Softmax attention with sinks.  `side_by_side` selects the variant that stands beside a delta rule in a parallel mixer (biases,
    per-head norm, halves layout, output gate); the other is the chunked one."""

    def __init__(self, width: int, m, eps: float, side_by_side: bool):
        super().__init__()
        h, d = int(_get(m, "heads")), int(_get(m, "dim"))
        g, dv = int(_get(m, "kv_heads", h)), int(_get(m, "vdim", d))
        rot, mask = _get(m, "rot"), _get(m, "mask")
        rot_dims = int(_get(rot, "dims", d)) if rot else 0
        freq = banded_frequencies(rot_dims, float(_get(rot, "base", 10000.0)), _get(rot, "scaling")) if rot_dims else None
        self.proj = MergedLinear(width, [h * d, g * d, g * dv] + ([h] if side_by_side else []), ["q", "k", "v"] + (["g"] if side_by_side else []),
                                 bias=side_by_side)
        self.attn = GatedValueRotaryAttention(h, g, d, dv, float(_get(m, "scale", d ** -0.5)), eps, rot_dims, freq, 1.0, None, gated=side_by_side,
                                              interleaved=not side_by_side, norm_per_head=side_by_side, chunk=int(_get(mask, "size", 0) or 0) if mask else 0,
                                              sinks=True)
        self.o = MergedLinear(h * dv, [width])

    def forward(self, x: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        return self.o(self.attn(self.proj(x), positions))


class SokipelDelta(nn.Module):
    def __init__(self, width: int, m, eps: float):
        super().__init__()
        h, d = int(_get(m, "heads")), int(_get(m, "dim"))
        g, dv = int(_get(m, "kv_heads", h)), int(_get(m, "vdim", d))
        self.cell = GatedDeltaRule(h, g, d, dv, int(_get(m, "conv", 1)), eps)
        nq, nk, nv, nb, na, ng = self.cell.projection_sizes()
        # (the gate's columns follow the convolved ones, the two narrow per-head blocks come last: wide blocks stay aligned)
        self.proj = MergedLinear(width, [nq, nk, nv, ng, nb, na], ["q", "k", "v", "g", "b", "a"])
        self.columns = [nq + nk + nv, ng, nb, na]            # q | k | v adjoin: one view for the convolution
        self.o = MergedLinear(h * dv, [width])

    def forward(self, x: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        qkv, gate, b, a = self.proj(x).split(self.columns, dim=-1)
        return self.o(self.cell(qkv, b, a, gate))


class SokipelParallelMixer(nn.Module):
    """left_scale * attention(h) + right_scale * delta(h); the sum is formed inside the layer's closing kernel (forward names its terms)."""

    def __init__(self, width: int, m, eps: float):
        super().__init__()
        self.left = SokipelAttention(width, _get(m, "left"), eps, side_by_side=True)
        self.right = SokipelDelta(width, _get(m, "right"), eps)
        self.left_scale, self.right_scale = float(_get(m, "left_scale", 1.0)), float(_get(m, "right_scale", 1.0))

    def forward(self, x: torch.Tensor, positions: torch.Tensor) -> dict:
        return dict(a=self.left(x, positions), a_scale=self.left_scale, b=self.right(x, positions), b_scale=self.right_scale)


class SokipelLayer(nn.Module):
    def __init__(self, width: int, spec, eps: float, mult: float, taps: int):
        super().__init__()
        kind, mixer, mlp = _get(spec, "type"), _get(spec, "mixer"), _get(spec, "mlp")
        self.canon = StreamConv(width, taps) if taps else None
        if kind == "attention":
            self.mixer = SokipelAttention(width, mixer, eps, side_by_side=False)
        elif kind == "delta":
            self.mixer = SokipelDelta(width, mixer, eps)
        elif kind == "parallel":
            self.mixer = SokipelParallelMixer(width, mixer, eps)
        else:
            raise ValueError(f"unknown mixer type {kind!r}")
        self.norm1 = SublayerOutputNorm(eps, mult)
        self.mlp = None
        if mlp:
            if _get(mlp, "kind", "moe") != "moe":
                raise ValueError(f"unknown feed-forward kind {_get(mlp, 'kind')!r}")
            expert, router = _get(mlp, "expert"), _get(mlp, "router")
            self.mlp = SparseMoE(width, int(_get(expert, "ff")), int(_get(router, "experts")), int(_get(router, "top")), act="glu_clamp",
                                 router_bias=False, score="sigmoid", limit=float(_get(expert, "limit")), weight_on_input=True)
            self.norm2 = SublayerOutputNorm(eps, mult)


class SokipelForCausalLM(nn.Module):
    requires_cache = True            # attention reads its keys from the paged cache in every step (no packed mode)
    has_recurrent_state = True       # sequences hold a state slot; cached pages cannot stand in for a prefix
    supported_dtypes = (torch.bfloat16, torch.float32)

    def __init__(self, config) -> None:
        super().__init__()
        self.config = config
        width, vocab = int(config.width), int(config.vocab)
        eps = float(_get(config.norm, "eps", 1e-6))
        mult = float(getattr(config, "residual_mult", 1.0))
        canon = getattr(config, "canon", None)
        taps = int(_get(canon, "taps", 0) or 0) if canon else 0
        self.width, self.vocab = width, vocab
        self.embed_scale = float(_get(getattr(config, "embedding", None) or {}, "scale", 1.0))
        self.softcap = float(getattr(config, "logit_softcap", 0.0) or 0.0)
        self.embed = MergedLinear(width, [vocab])            # [vocab, width]: a table, stored like a projection
        self.layers = nn.ModuleList([SokipelLayer(width, spec, eps, mult, taps) for spec in config.layers])
        self.final_norm = StreamNorm(width, eps, "rms")      # the checkpoint holds one number: it is spread over the columns at load time
        self.final_norm.weight.weight_loader = lambda param, t: param.data.copy_(t.reshape(-1).expand(param.shape[0]) if t.numel() == 1 else t)
        self.head = MergedLinear(width, [vocab])
        self.collect = None          # a list: receives a copy of the stream after every layer (debugging, tests)

    # ------------------------------------------------------------------ checkpoint names
    def weight_target(self, name: str):
        """(parameter name, shard id | None) of a checkpoint tensor."""
        top = {"embed": "embed.weight", "head": "head.weight", "final.norm": "final_norm.weight"}
        if name in top:
            return top[name], None
        m = re.fullmatch(r"l(\d+)\.(.+)", name)
        if not m:
            raise KeyError(f"checkpoint tensor {name!r} matches no parameter of the model")
        i, rest = int(m.group(1)), m.group(2)
        p = f"layers.{i}."
        direct = {"norm1": "norm1.weight", "norm2": "norm2.weight", "canon1": "canon.weight"}
        if rest in direct:
            return p + direct[rest], None
        if rest.startswith("mlp."):
            leaf = rest[4:]
            if leaf == "router":
                return p + "mlp.router.weight", None
            e = re.fullmatch(r"e(\d+)\.(gate|up|down)", leaf)
            if e:
                n = int(e.group(1))
                return (p + "mlp.down", n) if e.group(2) == "down" else (p + "mlp.gate_up", (n, e.group(2)))
        elif rest.startswith("mix."):
            leaf, pm, mixer = rest[4:], p + "mixer.", self.layers[i].mixer
            if isinstance(mixer, SokipelParallelMixer):
                side, _, leaf = leaf.partition(".")
                if side in ("left", "right"):
                    pm, mixer = pm + side + ".", getattr(mixer, side)
            target = self._mixer_target(mixer, pm, leaf)
            if target is not None:
                return target
        raise KeyError(f"checkpoint tensor {name!r} matches no parameter of the model")

    @staticmethod
    def _mixer_target(mixer, pm: str, leaf: str):
        if leaf == "o":
            return pm + "o.weight", None
        if isinstance(mixer, SokipelAttention):
            direct = {"q.norm": "attn.q_norm", "k.norm": "attn.k_norm", "sink": "attn.sinks"}
            if leaf in direct:
                return pm + direct[leaf], None
            if leaf in mixer.proj.shard_ids:
                return pm + "proj.weight", leaf
            if leaf.endswith(".b") and leaf[:-2] in mixer.proj.shard_ids and mixer.proj.bias is not None:
                return pm + "proj.bias", leaf[:-2]
        elif isinstance(mixer, SokipelDelta):
            direct = {"A_log": "cell.A_log", "dt_bias": "cell.dt_bias", "norm": "cell.norm"}
            if leaf in direct:
                return pm + direct[leaf], None
            if leaf in mixer.proj.shard_ids:
                return pm + "proj.weight", leaf
            if leaf.endswith(".conv") and leaf[:-5] in ("q", "k", "v"):
                return pm + "cell.conv_weight", leaf[:-5]
        return None

    @staticmethod
    def synthetic_tensors(config, seed: int = 0, std: float = 0.02, device="cuda", dtype=torch.bfloat16):
        """Random weights in checkpoint naming (for benchmarks and smoke runs without a checkpoint)."""
        width, vocab = int(config.width), int(config.vocab)
        canon = getattr(config, "canon", None)
        taps = int(_get(canon, "taps", 0) or 0) if canon else 0

        def mat(name, *shape, scale=std, shift=0.0):
            g = torch.Generator(device=device)
            g.manual_seed((zlib.crc32(name.encode()) ^ (seed * 0x9E3779B1)) & 0x7FFFFFFF)
            return name, (torch.randn(tuple(shape), generator=g, device=device, dtype=torch.float32) * scale + shift).to(dtype)

        def attention(p, m, side_by_side):
            h, d = int(_get(m, "heads")), int(_get(m, "dim"))
            g, dv = int(_get(m, "kv_heads", h)), int(_get(m, "vdim", d))
            for leaf, n in (("q", h * d), ("k", g * d), ("v", g * dv)):
                yield mat(p + leaf, n, width)
                if side_by_side:
                    yield mat(p + leaf + ".b", n, scale=0.1)
            yield mat(p + "q.norm", d if side_by_side else h * d, scale=0.1, shift=1.0)
            yield mat(p + "k.norm", d if side_by_side else g * d, scale=0.1, shift=1.0)
            yield mat(p + "sink", h, scale=1.0)
            if side_by_side:
                yield mat(p + "g", h, width)
            yield mat(p + "o", width, h * dv)

        def delta(p, m):
            h, d = int(_get(m, "heads")), int(_get(m, "dim"))
            g, dv, conv = int(_get(m, "kv_heads", h)), int(_get(m, "vdim", d)), int(_get(m, "conv", 1))
            for leaf, n in (("q", g * d), ("k", g * d), ("v", h * dv)):
                yield mat(p + leaf, n, width)
                yield mat(p + leaf + ".conv", n, conv, scale=0.4)
            yield mat(p + "b", h, width)
            yield mat(p + "a", h, width)
            yield mat(p + "A_log", h, scale=0.5)
            yield mat(p + "dt_bias", h, scale=0.5, shift=-2.0)
            yield mat(p + "norm", dv, scale=0.1, shift=1.0)
            yield mat(p + "g", h * dv, width)
            yield mat(p + "o", width, h * dv)

        yield mat("embed", vocab, width, scale=1.0)
        yield mat("head", vocab, width)
        yield mat("final.norm", scale=0.1, shift=1.0)
        for i, spec in enumerate(config.layers):
            p, m, kind = f"l{i}.", _get(spec, "mixer"), _get(spec, "type")
            yield mat(p + "norm1", scale=0.1, shift=1.0)
            if taps:
                yield mat(p + "canon1", width, taps, scale=0.2)
            if kind == "attention":
                yield from attention(p + "mix.", m, False)
            elif kind == "delta":
                yield from delta(p + "mix.", m)
            else:
                yield from attention(p + "mix.left.", _get(m, "left"), True)
                yield from delta(p + "mix.right.", _get(m, "right"))
            mlp = _get(spec, "mlp")
            if not mlp:
                continue
            yield mat(p + "norm2", scale=0.1, shift=1.0)
            ff, experts = int(_get(_get(mlp, "expert"), "ff")), int(_get(_get(mlp, "router"), "experts"))
            for e in range(experts):
                yield mat(f"{p}mlp.e{e}.gate", ff, width)
                yield mat(f"{p}mlp.e{e}.up", ff, width)
                yield mat(f"{p}mlp.e{e}.down", width, ff)
            yield mat(p + "mlp.router", experts, width)

    # ------------------------------------------------------------------ forward
    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        """The fp32 residual stream [T, width] after the last layer (the final norm runs on the rows that are projected)."""
        table = self.embed.weight.data
        x = ops.embedding_pos_stream(input_ids, positions, table, None, self.embed_scale)
        h = None                                             # the stream in the activation type, where the next reader wants it as it is
        last = len(self.layers) - 1
        for i, layer in enumerate(self.layers):
            if layer.canon is not None:
                h = layer.canon(x)
            elif h is None:
                h = torch.empty(x.shape, dtype=table.dtype, device=x.device)
                ops.stream_cast_(x, h)
            terms = layer.mixer(h, positions)
            if not isinstance(terms, dict):
                terms = dict(a=terms)
            plain_next = i < last and self.layers[i + 1].canon is None
            h = layer.norm1.close(x, **terms, want_h=layer.mlp is not None or plain_next)
            if layer.mlp is not None:
                h = layer.norm2.close(x, c32=layer.mlp(h), want_h=plain_next)
            if self.collect is not None:
                self.collect.append(x.clone())
        return x

    def gather_rows(self, hidden: torch.Tensor, rows: torch.Tensor) -> torch.Tensor:
        return ops.gather_rows_f32(hidden, rows)

    def compute_logits_rows(self, rows: torch.Tensor) -> torch.Tensor:
        """fp32 logits [R, vocab] of selected rows of the stream: final norm, head, softcap."""
        return ops.logits_scale(self.head(self.final_norm(rows), out_f32=True), 1.0, self.softcap)

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        return self.compute_logits_rows(hidden)
