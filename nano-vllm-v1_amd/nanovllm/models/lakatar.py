"""Lakatar: a decoder-only stack that norms AFTER every residual sum, over an fp32 residual stream, with three kinds of sequence
mixers (retention, an RWKV-style time mix, softmax attention through a low-rank latent) and mixture-of-experts feed-forwards.

    x = embed[token]
    for every layer:
        x = norm1(alpha x + ls1 * mixer(x))          (RMS norm with weight 1 + w; ls: a per-column layer scale; the sublayers read x itself)
        x = norm2(alpha x + ls2 * ff(x))             (layers without a feed-forward skip this)
    logits = head(final_norm(x))

Mixers (sizes and constants per layer from config.json):
  retention         q, k, v, gate from one merged projection; rotary (halves layout) on q and k, k / sqrt(dim); one fixed decay per head;
                    per-head unit read-out times silu(gate)  (layers.recurrent.Retention)
  wkv               the previous token's input blended into five inputs (layers.recurrent.TokenShift); r, k, v, gate and a low-rank
                    decay logit, each from its own blend; matrix memory read before it is written, with a bonus for the token itself
                    (layers.recurrent.WKV)
  latent_attention  queries through a normed latent; keys and values from ONE cached normed latent and one cached rotated key part
                    shared by the heads (interleaved rotary, YaRN-scaled frequencies); per-head sigmoid output gate
                    (layers.attention.LatentAttention).  A layer with `kv_from: j` reads the latent that layer j cached.
Feed-forward: layers.moe.SparseMoE with score="softmax_all": softmax scores, a correction that steers the choice only, groups of
experts of which the best stay eligible, scaled unnormalised weights, a shared expert behind a sigmoid gate per token.

32-bit whatever the activation type: the residual stream, its sums and norms, rotary angles, attention scores and weights, router
logits, scores and weights, every operand of a recurrence (decays, the bonus, the state, the read-out norms).  Projections and
their activations run in the model's dtype (bf16, or fp32 for a model served in full precision).

config.json keys: architecture, vocab, width, norm.eps, postln_alpha, layers[] of {type, mixer {...}, mlp {kind: moe, expert {ff},
router {experts, top, scale, groups {count, keep} | null}, shared {ff} | null} | null}.  retention mixer: heads, dim, vdim, decay[],
rot {base, dims, scaling | null}; wkv: heads, dim; latent_attention: heads, dim, rot_dim, vdim, q_rank, kv_rank, scale,
rot {base, dims, scaling {factor, original, fast, slow} | null}, kv_from | null.  Tensors: embed, head, final.norm,
l<i>.norm1|norm2|ls1|ls2, l<i>.mix.*, l<i>.mlp.e<n>.gate|up|down, l<i>.mlp.router|correction, l<i>.mlp.shared.gate|up|down|sg.
"""
from __future__ import annotations

import re
import zlib

import torch
from torch import nn

from .. import ops
from ..layers.attention import LatentAttention
from ..layers.layernorm import PostSumRMSNorm
from ..layers.linear import MergedLinear
from ..layers.moe import SparseMoE
from ..layers.recurrent import WKV, Retention, TokenShift
from ..layers.rotary_embedding import rotary_frequencies
from .lamutar import _get


class LakatarRetention(nn.Module):
    def __init__(self, width: int, m, eps: float):
        super().__init__()
        h, d = int(_get(m, "heads")), int(_get(m, "dim"))
        dv = int(_get(m, "vdim", d))
        rot = _get(m, "rot")
        rot_dims = int(_get(rot, "dims", d)) if rot else 0
        freq, mag = rotary_frequencies(rot_dims, float(_get(rot, "base", 10000.0)), _get(rot, "scaling")) if rot_dims else (None, 1.0)
        self.proj = MergedLinear(width, [h * d, h * d, h * dv, h * dv], ["q", "k", "v", "g"])
        self.cell = Retention(h, d, dv, [float(x) for x in _get(m, "decay")], eps, rot_dims, freq, mag, interleaved=False)
        self.o = MergedLinear(h * dv, [width])

    def forward(self, x: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        q, k, v, g = self.proj.split(self.proj(x))
        return self.o(self.cell(q, k, v, g, positions))


class LakatarWkv(nn.Module):
    MIXES = ("r", "k", "v", "g", "w")            # the consumers of the token shift, in the order of its rows

    def __init__(self, width: int, m, eps: float, rank: int):
        super().__init__()
        h, d = int(_get(m, "heads")), int(_get(m, "dim"))
        n = h * d
        self.shift = TokenShift(width, len(self.MIXES))
        self.shift.mu.shard_ids = list(self.MIXES)
        self.shift.mu.weight_loader = lambda param, t, shard: param.data[self.MIXES.index(shard)].copy_(t)
        self.r, self.k, self.v, self.g = (MergedLinear(width, [n]) for _ in range(4))
        self.w1 = MergedLinear(width, [rank])
        self.cell = WKV(h, d, rank, eps)
        self.o = MergedLinear(n, [width])

    def forward(self, x: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        mr, mk, mv, mg, mw = self.shift(x)
        return self.o(self.cell(self.r(mr), self.k(mk), self.v(mv), self.g(mg), self.w1(mw)))


class LakatarLatentAttention(nn.Module):
    def __init__(self, width: int, m, eps: float, source: "LakatarLatentAttention | None"):
        super().__init__()
        h, d, dr = int(_get(m, "heads")), int(_get(m, "dim")), int(_get(m, "rot_dim"))
        dv, rq, rkv = int(_get(m, "vdim", d)), int(_get(m, "q_rank")), int(_get(m, "kv_rank"))
        rot = _get(m, "rot")
        assert dr == 0 or int(_get(rot, "dims", dr)) == dr, "the rotated part is the whole of rot_dim"
        freq, mag = rotary_frequencies(dr, float(_get(rot, "base", 10000.0)), _get(rot, "scaling")) if dr else (None, 1.0)
        self.attn = LatentAttention(h, d, dr, dv, rq, rkv, float(_get(m, "scale", (d + dr) ** -0.5)), eps, freq, mag, interleaved=True, gated=True,
                                    kv_source=None if source is None else source.attn)
        names = ["dq"] + ([] if source is not None else ["dkv"]) + ["g"]
        self.proj = MergedLinear(width, self.attn.projection_sizes(), names)
        self.o = MergedLinear(h * dv, [width])

    def forward(self, x: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        return self.o(self.attn(self.proj(x), positions))


class LakatarMoE(nn.Module):
    def __init__(self, width: int, mlp):
        super().__init__()
        router, shared, groups = _get(mlp, "router"), _get(mlp, "shared"), _get(_get(mlp, "router"), "groups")
        self.moe = SparseMoE(width, int(_get(_get(mlp, "expert"), "ff")), int(_get(router, "experts")), int(_get(router, "top")),
                             shared_ff=int(_get(shared, "ff")) if shared else None, act="silu", router_bias=False, score="softmax_all", correction=True,
                             groups=int(_get(groups, "count", 1)) if groups else 1, keep_groups=int(_get(groups, "keep", 1)) if groups else 1,
                             route_scale=float(_get(router, "scale", 1.0)), shared_gate=bool(shared))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.moe(x)


class LakatarLayer(nn.Module):
    def __init__(self, width: int, spec, eps: float, alpha: float, rank: int, latents: dict, index: int):
        super().__init__()
        kind, mixer, mlp = _get(spec, "type"), _get(spec, "mixer"), _get(spec, "mlp")
        if kind == "retention":
            self.mixer = LakatarRetention(width, mixer, eps)
        elif kind == "wkv":
            self.mixer = LakatarWkv(width, mixer, eps, rank)
        elif kind == "latent_attention":
            src = _get(mixer, "kv_from")
            if src is not None and int(src) not in latents:
                raise ValueError(f"layer {index} takes its latent from layer {src}, which is no earlier latent-attention layer with a latent of its own")
            self.mixer = LakatarLatentAttention(width, mixer, eps, None if src is None else latents[int(src)])
            if src is None:
                latents[index] = self.mixer
        else:
            raise ValueError(f"unknown mixer type {kind!r}")
        self.norm1 = PostSumRMSNorm(width, eps, alpha, weight_offset=1.0, layer_scale=True)
        self.mlp = None
        if mlp:
            if _get(mlp, "kind", "moe") != "moe":
                raise ValueError(f"unknown feed-forward kind {_get(mlp, 'kind')!r}")
            self.mlp = LakatarMoE(width, mlp)
            self.norm2 = PostSumRMSNorm(width, eps, alpha, weight_offset=1.0, layer_scale=True)


class LakatarForCausalLM(nn.Module):
    requires_cache = True            # attention reads its keys from the paged cache in every step (no packed mode)
    has_recurrent_state = True       # sequences hold a state slot; cached pages cannot stand in for a prefix
    supported_dtypes = (torch.bfloat16, torch.float32)
    DEFAULT_DECAY_RANK = 16

    def __init__(self, config) -> None:
        super().__init__()
        self.config = config
        width, vocab = int(config.width), int(config.vocab)
        eps = float(_get(config.norm, "eps", 1e-6))
        alpha = float(getattr(config, "postln_alpha", 1.0))
        self.width, self.vocab = width, vocab
        ranks = getattr(config, "decay_ranks", None) or {}
        self.embed = MergedLinear(width, [vocab])            # [vocab, width]: a table, stored like a projection
        latents: dict = {}
        self.layers = nn.ModuleList([LakatarLayer(width, spec, eps, alpha, ranks.get(i, self.DEFAULT_DECAY_RANK), latents, i)
                                     for i, spec in enumerate(config.layers)])
        self.final_norm = PostSumRMSNorm(width, eps, 1.0, weight_offset=1.0)
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
        direct = {"norm1": "norm1.weight", "norm2": "norm2.weight", "ls1": "norm1.scale", "ls2": "norm2.scale"}
        if rest in direct:
            return p + direct[rest], None
        if rest.startswith("mlp."):
            return self._mlp_target(p + "mlp.moe.", rest[4:], name)
        if not rest.startswith("mix."):
            raise KeyError(f"checkpoint tensor {name!r} matches no parameter of the model")
        leaf, pm, mixer = rest[4:], p + "mixer.", self.layers[i].mixer
        if leaf == "o":
            return pm + "o.weight", None
        if isinstance(mixer, LakatarRetention):
            if leaf in ("q", "k", "v", "g"):
                return pm + "proj.weight", leaf
        elif isinstance(mixer, LakatarWkv):
            if leaf.startswith("mu.") and leaf[3:] in LakatarWkv.MIXES:
                return pm + "shift.mu", leaf[3:]
            if leaf in ("r", "k", "v", "g", "w1"):
                return pm + leaf + ".weight", None
            direct = {"w2": "cell.w2", "w0": "cell.w0", "u": "cell.bonus", "norm": "cell.norm"}
            if leaf in direct:
                return pm + direct[leaf], None
        elif isinstance(mixer, LakatarLatentAttention):
            if leaf in ("dq", "dkv", "g"):
                return pm + "proj.weight", leaf
            direct = {"dq.norm": "attn.q_norm", "dkv.norm": "attn.kv_norm", "uq": "attn.uq.weight", "uk": "attn.uk_t", "uv": "attn.uv"}
            if leaf in direct:
                return pm + direct[leaf], None
        raise KeyError(f"checkpoint tensor {name!r} matches no parameter of the model")

    @staticmethod
    def _mlp_target(p: str, leaf: str, name: str):
        direct = {"router": "router.weight", "correction": "correction", "shared.sg": "shared_gate.weight", "shared.down": "shared.down.weight"}
        if leaf in direct:
            return p + direct[leaf], None
        if leaf in ("shared.gate", "shared.up"):
            return p + "shared.gate_up.weight", leaf[7:]
        m = re.fullmatch(r"e(\d+)\.(gate|up|down)", leaf)
        if not m:
            raise KeyError(f"checkpoint tensor {name!r} matches no parameter of the model")
        e = int(m.group(1))
        return (p + "down", e) if m.group(2) == "down" else (p + "gate_up", (e, m.group(2)))

    @staticmethod
    def adapt_config(config, shapes: dict) -> None:
        """Sizes that only the checkpoint's tensor shapes give: the rank of each wkv layer's low-rank decay projection (`shapes`:
        tensor name -> shape; empty without a checkpoint, then the default rank is used)."""
        ranks = {}
        for name, shape in shapes.items():
            m = re.fullmatch(r"l(\d+)\.mix\.w1", name)
            if m:
                ranks[int(m.group(1))] = int(shape[0])
        config.decay_ranks = ranks

    @staticmethod
    def synthetic_tensors(config, seed: int = 0, std: float = 0.02, device="cuda", dtype=torch.bfloat16):
        """Random weights in checkpoint naming (for benchmarks and smoke runs without a checkpoint)."""
        width, vocab = int(config.width), int(config.vocab)
        ranks = getattr(config, "decay_ranks", None) or {}

        def mat(name, *shape, scale=std, shift=0.0):
            g = torch.Generator(device=device)
            g.manual_seed((zlib.crc32(name.encode()) ^ (seed * 0x9E3779B1)) & 0x7FFFFFFF)
            return name, (torch.randn(*shape, generator=g, device=device, dtype=torch.float32) * scale + shift).to(dtype)

        yield mat("embed", vocab, width, scale=1.0)
        yield mat("head", vocab, width)
        yield mat("final.norm", width, scale=0.1)
        for i, spec in enumerate(config.layers):
            p, m, kind = f"l{i}.", _get(spec, "mixer"), _get(spec, "type")
            yield mat(p + "norm1", width, scale=0.1)
            yield mat(p + "ls1", width, scale=0.1, shift=1.0)
            h, d = int(_get(m, "heads")), int(_get(m, "dim"))
            if kind == "retention":
                dv = int(_get(m, "vdim", d))
                for leaf, n in (("q", h * d), ("k", h * d), ("v", h * dv), ("g", h * dv)):
                    yield mat(p + "mix." + leaf, n, width)
                yield mat(p + "mix.o", width, h * dv)
            elif kind == "wkv":
                n, rank = h * d, ranks.get(i, LakatarForCausalLM.DEFAULT_DECAY_RANK)
                for leaf in LakatarWkv.MIXES:
                    yield mat(p + "mix.mu." + leaf, width, scale=0.2, shift=0.5)
                for leaf in ("r", "k", "v", "g"):
                    yield mat(p + "mix." + leaf, n, width)
                yield mat(p + "mix.w1", rank, width)
                yield mat(p + "mix.w2", n, rank, scale=0.1)
                yield mat(p + "mix.w0", n, scale=1.0, shift=-2.0)
                yield mat(p + "mix.u", h, d, scale=0.3)
                yield mat(p + "mix.norm", n, scale=0.1, shift=1.0)
                yield mat(p + "mix.o", width, n)
            else:
                dr, dv, rq, rkv = int(_get(m, "rot_dim")), int(_get(m, "vdim", d)), int(_get(m, "q_rank")), int(_get(m, "kv_rank"))
                yield mat(p + "mix.dq", rq, width)
                yield mat(p + "mix.dq.norm", rq, scale=0.1, shift=1.0)
                yield mat(p + "mix.uq", h * (d + dr), rq)
                if _get(m, "kv_from") is None:
                    yield mat(p + "mix.dkv", rkv + dr, width)
                    yield mat(p + "mix.dkv.norm", rkv, scale=0.1, shift=1.0)
                yield mat(p + "mix.uk", h * d, rkv)
                yield mat(p + "mix.uv", h * dv, rkv)
                yield mat(p + "mix.g", h, width)
                yield mat(p + "mix.o", width, h * dv)
            mlp = _get(spec, "mlp")
            if not mlp:
                continue
            yield mat(p + "norm2", width, scale=0.1)
            yield mat(p + "ls2", width, scale=0.1, shift=1.0)
            ff, router, shared = int(_get(_get(mlp, "expert"), "ff")), _get(mlp, "router"), _get(mlp, "shared")
            experts = int(_get(router, "experts"))
            for e in range(experts):
                yield mat(f"{p}mlp.e{e}.gate", ff, width)
                yield mat(f"{p}mlp.e{e}.up", ff, width)
                yield mat(f"{p}mlp.e{e}.down", width, ff)
            yield mat(p + "mlp.router", experts, width)
            yield mat(p + "mlp.correction", experts, scale=0.05)
            if shared:
                sf = int(_get(shared, "ff"))
                yield mat(p + "mlp.shared.gate", sf, width)
                yield mat(p + "mlp.shared.up", sf, width)
                yield mat(p + "mlp.shared.down", width, sf)
                yield mat(p + "mlp.shared.sg", 1, width)

    # ------------------------------------------------------------------ forward
    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        """The fp32 residual stream [T, width] after the last layer (the final norm runs on the rows that are projected)."""
        table = self.embed.weight.data
        h = torch.empty(input_ids.numel(), self.width, dtype=table.dtype, device=table.device)
        x = ops.embedding_stream(input_ids, table, h)         # the stream in fp32 and, in the activation type, the first sublayer's input
        for layer in self.layers:
            h = layer.norm1.close(x, y=layer.mixer(h, positions))
            if layer.mlp is not None:
                h = layer.norm2.close(x, y32=layer.mlp(h))
            if self.collect is not None:
                self.collect.append(x.clone())
        return x

    def gather_rows(self, hidden: torch.Tensor, rows: torch.Tensor) -> torch.Tensor:
        return ops.gather_rows_f32(hidden, rows)

    def compute_logits_rows(self, rows: torch.Tensor) -> torch.Tensor:
        """fp32 logits [R, vocab] of selected rows of the stream: final norm, head."""
        return self.head(self.final_norm(rows), out_f32=True)

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        return self.compute_logits_rows(hidden)
