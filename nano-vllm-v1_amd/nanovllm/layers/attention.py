"""Paged attention operator module (reference interface: nanovllm/layers/attention.py:93-249).

``Attention(num_heads, head_dim, scale, num_kv_heads)`` with ``k_cache`` / ``v_cache``
attributes that the runner binds to per-layer views [pages, 256, Hkv, D] of the KV pool, and
``forward(q, k, v) -> o`` reading the per-step Context:

  cu_seqlens_q is None        one query per sequence over the cache (graph-replay decode)
                              -> nvh_attn_decode (csrc/attention_decode.hip)
  block_tables is not None    var-len queries over the paged cache (chunked prefill, prefix
                              hits, mixed batches, eager decode) -> nvh_attn_varlen, or
                              nvh_attn_decode when every sequence has exactly one query
  block_tables is None        var-len self-attention over the packed new tokens (warm-up,
                              fresh un-chunked prefill) -> nvh_attn_varlen

New K/V rows are written to the cache first (nvh_store_kvcache) whenever a cache is bound.
"""
import torch
from torch import nn

from .. import ops
from ..utils.context import get_context
from .linear import MergedLinear


def store_kvcache(key: torch.Tensor, value: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                  slot_mapping: torch.Tensor) -> None:
    """key/value [N, Hkv, D] (token stride free) -> cache rows slot_mapping[n]; -1 skips."""
    ops.store_kvcache(key, value, k_cache, v_cache, slot_mapping)


class Attention(nn.Module):
    def __init__(self, num_heads, head_dim, scale, num_kv_heads):
        super().__init__()
        self.num_heads = num_heads
        self.head_dim = head_dim
        self.scale = scale
        self.num_kv_heads = num_kv_heads
        self.k_cache = self.v_cache = torch.tensor([])
        self.decode_splits = 0          # 0 = heuristic per call
        self.max_context = None
        self.split_fn = None            # (batch, longest context) -> (key ranges, minimum keys per range); the runner
                                        # installs one policy for eager and graph steps

    def attend(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
        """Attention proper, with the new K/V already in the cache (or no cache bound)."""
        ctx = get_context()
        splits, min_range = (self.split_fn(q.shape[0], ctx.max_seqlen_k or 0) if self.split_fn is not None
                             else (self.decode_splits, 0))
        if ctx.cu_seqlens_q is None:
            return ops.attn_decode(q, self.k_cache, self.v_cache, ctx.context_lens, ctx.block_tables, self.scale,
                                   splits, self.max_context, min_range)
        if ctx.block_tables is not None:
            if ctx.max_seqlen_q == 1 and ctx.context_lens is not None:
                return ops.attn_decode(q, self.k_cache, self.v_cache, ctx.context_lens, ctx.block_tables, self.scale,
                                       splits, ctx.max_seqlen_k, min_range)
            return ops.attn_varlen(q, self.k_cache, self.v_cache, ctx.cu_seqlens_q, ctx.cu_seqlens_k,
                                   ctx.max_seqlen_q, self.scale, ctx.block_tables, ctx.max_seqlen_k or None)
        return ops.attn_varlen(q, k, v, ctx.cu_seqlens_q, ctx.cu_seqlens_k, ctx.max_seqlen_q, self.scale,
                               None, ctx.max_seqlen_k or None)

    def forward(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
        ctx = get_context()
        if self.k_cache.numel() and self.v_cache.numel() and ctx.slot_mapping is not None and ctx.slot_mapping.numel():
            store_kvcache(k, v, self.k_cache, self.v_cache, ctx.slot_mapping)
        return self.attend(q, k, v)


class GatedValueRotaryAttention(nn.Module):
    """Paged causal attention with free head sizes (query/key `head_dim`, value `value_dim`), a partial rotary on q/k
    whose frequencies the caller supplies, optionally values that are rotated by their own position before they are
    cached (each head's output is turned back by the query's position), and optionally a per-head sigmoid output gate.

    Input is the fused projection output [T, H*dim + G*dim + G*vdim (+ H)] = q | k | v | gate; RMS norms over the WHOLE
    q and k projections (or, with `norm_per_head`, over every head by itself with a weight row [dim] that the heads share) run
    with the rotary in one launch (nvh_attn_rotary_prep), attention in a second (nvh_attn_paged_any).  `chunk` > 0: a query
    sees only the earlier tokens of its own block of `chunk` positions, blocks counted from the sequence's start.  `sinks`: a
    learned logit per head (parameter `sinks`, fp32) is one more term exp(sink) of the softmax's denominator - it stands for no
    token, carries no value and is taken as it is, without `scale` - so a head can give weight to nothing.  A module that serves several passes of a looped stack
    owns one cache per pass:
    `k_caches[run]` [pages, page, G, dim] and `v_caches[run]` [pages, G, vdim, page] (values lie transposed within a page),
    bound by the runner (`cache_runs` of each)."""

    def __init__(self, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int, scale: float, eps: float,
                 rot_dims: int, qk_freq: torch.Tensor | None, qk_mag: float, value_freq: torch.Tensor | None, gated: bool,
                 cache_runs: int = 1, interleaved: bool = False, norm_per_head: bool = False, chunk: int = 0, sinks: bool = False):
        super().__init__()
        assert num_heads % num_kv_heads == 0 and chunk >= 0 and (rot_dims == 0 or qk_freq is not None)
        self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim = num_heads, num_kv_heads, head_dim, value_dim
        self.scale, self.eps, self.rot_dims, self.qk_mag, self.gated, self.interleaved = scale, eps, rot_dims, qk_mag, gated, interleaved
        self.norm_per_head, self.chunk = norm_per_head, chunk
        self.q_norm = nn.Parameter(torch.ones(head_dim if norm_per_head else num_heads * head_dim), requires_grad=False)
        self.k_norm = nn.Parameter(torch.ones(head_dim if norm_per_head else num_kv_heads * head_dim), requires_grad=False)
        if sinks:
            self.sinks = nn.Parameter(torch.zeros(num_heads, dtype=torch.float32), requires_grad=False)      # (an operand of the fp32 softmax)
        else:
            self.register_parameter("sinks", None)
        self.register_buffer("qk_freq", None if qk_freq is None else qk_freq.to(dtype=torch.float32, device=self.q_norm.device), persistent=False)
        self.register_buffer("value_freq", None if value_freq is None else value_freq.to(dtype=torch.float32, device=self.q_norm.device),
                             persistent=False)
        self.cache_runs = cache_runs
        self.k_caches: list = [None] * cache_runs
        self.v_caches: list = [None] * cache_runs

    def cache_row_elems(self) -> tuple[int, int]:
        """Elements of one token's key row and value row (what the runner sizes the page pool with)."""
        return self.num_kv_heads * self.head_dim, self.num_kv_heads * self.value_dim

    def forward(self, proj: torch.Tensor, positions: torch.Tensor, run: int = 0) -> torch.Tensor:
        ctx = get_context()
        kc, vc = self.k_caches[run], self.v_caches[run]
        if kc is None or ctx.block_tables is None:
            raise RuntimeError("this attention reads its keys from the paged cache: bind caches and give every sequence a block table")
        q, gate = ops.attn_rotary_prep(proj, self.q_norm.data, self.k_norm.data, self.eps, positions, self.qk_freq, self.qk_mag,
                                       self.rot_dims, self.value_freq, kc, vc, ctx.slot_mapping, self.num_heads, self.num_kv_heads,
                                       self.head_dim, self.value_dim, self.gated, self.interleaved, self.interleaved, self.norm_per_head)
        return ops.attn_paged_any(q, kc, vc, ctx.cu_seqlens_q, ctx.context_lens, ctx.block_tables, self.scale, self.num_heads,
                                  self.num_kv_heads, self.head_dim, self.value_dim, gate, self.value_freq, self.interleaved, chunk=self.chunk,
                                  sinks=None if self.sinks is None else self.sinks.data)


class WindowedBiasAttention(nn.Module):
    """Paged causal attention without rotation whose scores carry a per-head distance bias, score = scale q.k - slope_h (i - j),
    and whose queries see a sliding window of the last `window` positions plus the first `keep_first` tokens of the sequence
    (window 0: every earlier token).  Free head sizes (query/key `head_dim`, value `value_dim`), grouped key/value heads.

    Input is the fused projection output [T, H*dim + G*dim + G*vdim] = q | k | v (biases already added).  k and v are
    scattered to their pages by nvh_attn_rotary_prep (no norm, no rotary), attention runs in nvh_attn_paged_any, which walks
    only the key tiles a query block can see.  The distance to a kept token is counted from where it really stands, so it
    grows.  Positions enter nowhere else, so the cache holds keys and values as projected.  One cache pair per pass of a
    looped stack (`cache_runs`), bound by the runner."""

    def __init__(self, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int, scale: float, slopes, window: int = 0,
                 keep_first: int = 0, cache_runs: int = 1):
        super().__init__()
        assert num_heads % num_kv_heads == 0 and window >= 0 and keep_first >= 0
        self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim = num_heads, num_kv_heads, head_dim, value_dim
        self.scale, self.window, self.keep_first = scale, window, keep_first
        slopes = None if slopes is None else torch.as_tensor(slopes, dtype=torch.float64).to(torch.float32)
        assert slopes is None or slopes.numel() == num_heads
        self.register_buffer("slopes", None if slopes is None else slopes.to(torch.empty(0).device), persistent=False)
        self.cache_runs = cache_runs
        self.k_caches: list = [None] * cache_runs
        self.v_caches: list = [None] * cache_runs

    @staticmethod
    def geometric_slopes(num_heads: int, span: float = 8.0) -> list[float]:
        """slope_h = 2^(-span (h + 1) / H), h = 0 .. H-1: the head-wise geometric sequence of linear distance biases."""
        return [2.0 ** (-span * (h + 1) / num_heads) for h in range(num_heads)]

    def cache_row_elems(self) -> tuple[int, int]:
        return self.num_kv_heads * self.head_dim, self.num_kv_heads * self.value_dim

    def forward(self, proj: torch.Tensor, positions: torch.Tensor, run: int = 0) -> torch.Tensor:
        ctx = get_context()
        kc, vc = self.k_caches[run], self.v_caches[run]
        if kc is None or ctx.block_tables is None:
            raise RuntimeError("this attention reads its keys from the paged cache: bind caches and give every sequence a block table")
        q, _ = ops.attn_rotary_prep(proj, None, None, 0.0, positions, None, 1.0, 0, None, kc, vc, ctx.slot_mapping, self.num_heads,
                                    self.num_kv_heads, self.head_dim, self.value_dim, gated=False)
        return ops.attn_paged_any(q, kc, vc, ctx.cu_seqlens_q, ctx.context_lens, ctx.block_tables, self.scale, self.num_heads,
                                  self.num_kv_heads, self.head_dim, self.value_dim, slopes=self.slopes, window=self.window,
                                  keep_first=self.keep_first)


class LatentAttention(nn.Module):
    """Causal softmax attention whose keys and values are read from a low-rank latent ("DeepSeek-V2: A Strong, Economical, and Efficient
    Mixture-of-Experts Language Model", DeepSeek-AI): a token leaves in the cache only its RMS-normed latent c (`kv_rank` wide) and
    one rotated key part k_r (`rot_dim` wide) that all heads share; head h's unrotated key is W_uk,h c and its value W_uv,h c.  Both are
    linear in c, so they are never formed: the query side takes W_uk in,

        score = scale ((W_uk,h^T q_n) . c + q_r . k_r),      out_h = W_uv,h (sum_j p_j c_j),

    which is paged attention of H query heads over ONE shared key/value head of key size kv_rank + rot_dim whose value is c
    (nvh_attn_paged_any), between two per-head products (nvh_gemm_heads_nt).  The query itself comes through a latent too
    (RMS-normed, `q_rank` wide) and is laid out per head as [dim unrotated | rot_dim rotated]; an optional sigmoid gate per head
    scales the head's output.

    Input of forward: the fused projection row [dq | dkv | gate] of the layer's input.  A module built with `kv_source` owns no
    cache and has no dkv part: it reads the latent and rotated key part that the source module cached for the same tokens (the
    source runs earlier in the step), with its own W_uk, W_uv and queries.  `uq` maps the normed query latent to the heads."""

    def __init__(self, num_heads: int, head_dim: int, rot_dim: int, value_dim: int, q_rank: int, kv_rank: int, scale: float, eps: float,
                 freq: torch.Tensor | None, mag: float = 1.0, interleaved: bool = True, gated: bool = True, cache_runs: int = 1,
                 kv_source: "LatentAttention | None" = None):
        super().__init__()
        self.num_heads, self.qk_dim, self.rot_dim, self.v_dim, self.q_rank, self.kv_rank = num_heads, head_dim, rot_dim, value_dim, q_rank, kv_rank
        self.scale, self.eps, self.mag, self.interleaved, self.gated = scale, eps, mag, interleaved, gated
        self.q_norm = nn.Parameter(torch.ones(q_rank), requires_grad=False)
        self.uq = MergedLinear(q_rank, [num_heads * (head_dim + rot_dim)])
        # W_uk is stored transposed per head ([H, kv_rank, dim]): it multiplies the query, not the latent
        self.uk_t = nn.Parameter(torch.empty(num_heads, kv_rank, head_dim), requires_grad=False)
        self.uk_t.weight_loader = self._load_uk
        self.uv = nn.Parameter(torch.empty(num_heads, value_dim, kv_rank), requires_grad=False)
        self.uv.weight_loader = self._load_uv
        self.register_buffer("freq", None if freq is None else freq.to(dtype=torch.float32, device=self.q_norm.device), persistent=False)
        self._source = [kv_source] if kv_source is not None else None       # (a list: the source is not a submodule of this one)
        if kv_source is None:
            self.kv_norm = nn.Parameter(torch.ones(kv_rank), requires_grad=False)
            self.cache_runs = cache_runs
            self.k_caches: list = [None] * cache_runs
            self.v_caches: list = [None] * cache_runs
        else:
            assert (kv_source.kv_rank, kv_source.rot_dim) == (kv_rank, rot_dim) and kv_source._source is None, "the source of a shared latent must own one of the same sizes"
            self.register_parameter("kv_norm", None)

    def _load_uk(self, param: nn.Parameter, loaded_weight: torch.Tensor):
        assert tuple(loaded_weight.shape) == (self.num_heads * self.qk_dim, self.kv_rank), tuple(loaded_weight.shape)
        param.data.copy_(loaded_weight.view(self.num_heads, self.qk_dim, self.kv_rank).transpose(1, 2))

    def _load_uv(self, param: nn.Parameter, loaded_weight: torch.Tensor):
        assert tuple(loaded_weight.shape) == (self.num_heads * self.v_dim, self.kv_rank), tuple(loaded_weight.shape)
        param.data.copy_(loaded_weight.view(self.num_heads, self.v_dim, self.kv_rank))

    # what the runner sizes and shapes the page pool with (modules without caches of their own are not asked)
    def cache_geometry(self) -> tuple[int, int, int]:
        """(key/value heads, key size, value size) of a cached token."""
        return 1, self.kv_rank + self.rot_dim, self.kv_rank

    def cache_row_elems(self) -> tuple[int, int]:
        return self.kv_rank + self.rot_dim, self.kv_rank

    def projection_sizes(self) -> list[int]:
        own = [] if self._source is not None else [self.kv_rank + self.rot_dim]
        return [self.q_rank] + own + ([self.num_heads] if self.gated else [])

    def forward(self, proj: torch.Tensor, positions: torch.Tensor, run: int = 0) -> torch.Tensor:
        ctx = get_context()
        owner = self if self._source is None else self._source[0]
        kc, vc = owner.k_caches[run], owner.v_caches[run]
        if kc is None or ctx.block_tables is None:
            raise RuntimeError("this attention reads its keys from the paged cache: bind caches and give every sequence a block table")
        own = self._source is None
        cq, gate = ops.latent_prep(proj, self.q_rank, self.kv_rank, self.rot_dim, self.num_heads, self.q_norm.data, self.kv_norm.data if own else None,
                                   self.eps, positions, self.freq, self.mag, self.interleaved, kc if own else None, vc if own else None,
                                   ctx.slot_mapping if own else None, self.gated)
        q = self.uq(cq)                                                     # [T, H * (dim + rot)]
        t, full = q.shape[0], self.kv_rank + self.rot_dim
        qa = torch.empty(t, self.num_heads * full, dtype=q.dtype, device=q.device)
        ops.linear_heads(q, self.uk_t.data, self.qk_dim + self.rot_dim, out=qa, out_head_stride=full)
        ops.latent_q_rotary(q, positions, self.freq, self.mag, self.interleaved, qa, self.num_heads, self.qk_dim, self.rot_dim, full, self.kv_rank)
        o = ops.attn_paged_any(qa, kc, vc, ctx.cu_seqlens_q, ctx.context_lens, ctx.block_tables, self.scale, self.num_heads, 1, full, self.kv_rank, gate)
        return ops.linear_heads(o, self.uv.data, self.kv_rank)
