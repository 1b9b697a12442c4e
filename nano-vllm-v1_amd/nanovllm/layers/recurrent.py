"""Recurrent mixers: layers that carry a fixed-size state per sequence instead of a growing cache.

The state of every live sequence sits in a slot of a pool [slots, ...] that the runner allocates and binds
(`states[run]`, one pool per pass of a looped stack); the step's Context names each sequence's slot (`state_slots`), and
a sequence whose tokens all arrive in this step starts from a zero state, whatever its slot held before.
"""
from __future__ import annotations

import math

import torch
from torch import nn

from .. import ops
from ..utils.context import get_context
from .linear import MergedLinear


class GeneralizedDeltaRule(nn.Module):
    """Per head a matrix memory S [dim, dim] in fp32, updated by every token:

        S <- diag(w) S - (a * u) (u^T S) + k v^T,      o = S^T r

    with a data-dependent decay w = exp(-decay_scale * sigmoid(w0 + W2 tanh(l))) in (0, 1) per key channel (l: a low-rank
    projection of the input), a removal rate a = sigmoid(a_raw + a_bias) along the unit key u = k / |k|, and the read-out
    normalised per head (o / rms(o) * norm) and gated by sigmoid(g).  `decay_scale` defaults to e^(-1/2).

    forward takes column views r, k, v, a_raw, g, l of the fused projection output and returns [T, H*dim] in the
    activation type, ready for the output projection (kernels: csrc/delta_rule.hip)."""

    def __init__(self, num_heads: int, head_dim: int, rank: int, eps: float, decay_scale: float = math.exp(-0.5), state_runs: int = 1):
        super().__init__()
        n = num_heads * head_dim
        self.num_heads, self.head_dim, self.rank, self.eps, self.decay_scale = num_heads, head_dim, rank, eps, decay_scale
        self.w2 = nn.Parameter(torch.zeros(n, rank), requires_grad=False)
        self.w0 = nn.Parameter(torch.zeros(n), requires_grad=False)
        self.a_bias = nn.Parameter(torch.zeros(n), requires_grad=False)
        self.norm = nn.Parameter(torch.ones(n), requires_grad=False)
        self.state_runs = state_runs
        self.states: list = [None] * state_runs

    def state_shape(self) -> tuple[int, int, int]:
        """Shape of one sequence's state (fp32 elements); the runner allocates [slots, *state_shape()] per run."""
        return self.num_heads, self.head_dim, self.head_dim

    def forward(self, r, k, v, a_raw, g, lowrank, run: int = 0) -> torch.Tensor:
        ctx = get_context()
        state = self.states[run]
        if state is None or ctx.state_slots is None:
            raise RuntimeError("the delta rule needs a bound state pool and a state slot per sequence")
        o = ops.delta_rule(r, k, v, a_raw, lowrank, self.w2.data, self.w0.data, self.a_bias.data, state, ctx.state_slots,
                           ctx.cu_seqlens_q, ctx.context_lens, self.num_heads, self.head_dim, self.decay_scale)
        return ops.delta_post(o, self.norm.data, g, self.num_heads, self.head_dim, self.eps)


class GatedDeltaRule(nn.Module):
    """The gated delta rule ("Gated Delta Networks: Improving Mamba2 with Delta Rule", Yang, Kautz, Hatamizadeh): per head a matrix memory
    S [key_dim, value_dim] in fp32 that decays as a whole and is corrected towards the token's value along its key,

        S <- g S;      d = beta (v - S^T k);      S <- S + k d^T;      o = S^T q          (o is taken after the update)

    with one decay g = exp(-exp(A_log) softplus(a + dt_bias)) and one write strength beta = sigmoid(b) per head and token.  q, k and v
    first pass a short causal convolution over time per channel (`taps` wide, last tap on the current token, no bias, continued across
    steps from the sequence's last taps - 1 inputs) and silu; q and k then become unit vectors per head, q also times key_dim^-1/2.
    q / k heads may be fewer than value heads: value head h reads q / k head h // (num_heads // qk_heads).  The read-out of a head is
    divided by its root mean square, multiplied by a weight row [value_dim] that the heads share, and by silu(gate).

    forward takes column views of the fused projection output - qkv (the convolved channels q | k | v, adjoining), b, a [T, H], gate
    [T, H * value_dim] - and returns [T, H * value_dim] in the activation type.  The scan is the generalized delta rule's
    (csrc/delta_rule.hip): g on every key channel, the removal along k at rate beta g, the written key beta k."""

    def __init__(self, num_heads: int, qk_heads: int, key_dim: int, value_dim: int, taps: int, eps: float, state_runs: int = 1):
        super().__init__()
        assert num_heads % qk_heads == 0 and taps >= 1
        self.num_heads, self.qk_heads, self.key_dim, self.value_dim, self.taps, self.eps = num_heads, qk_heads, key_dim, value_dim, taps, eps
        self.channel_sizes = [qk_heads * key_dim, qk_heads * key_dim, num_heads * value_dim]
        self.conv_weight = nn.Parameter(torch.zeros(sum(self.channel_sizes), taps), requires_grad=False)
        self.conv_weight.shard_ids = ["q", "k", "v"]
        self.conv_weight.weight_loader = self._load_conv
        self.dt_bias = nn.Parameter(torch.zeros(num_heads), requires_grad=False)
        self.A_log = nn.Parameter(torch.zeros(num_heads), requires_grad=False)
        self.norm = nn.Parameter(torch.ones(value_dim), requires_grad=False)
        self.conv_inputs = _StatePool((max(taps - 1, 1), sum(self.channel_sizes)), state_runs)     # the last taps - 1 inputs of q | k | v per sequence
        self.state_runs = state_runs
        self.states: list = [None] * state_runs

    def _load_conv(self, param: nn.Parameter, loaded_weight: torch.Tensor, shard_id):
        i = self.conv_weight.shard_ids.index(shard_id)
        dst = param.data.narrow(0, sum(self.channel_sizes[:i]), self.channel_sizes[i])
        assert dst.shape == loaded_weight.shape, f"convolution of {shard_id!r}: {tuple(loaded_weight.shape)} does not fit {tuple(dst.shape)}"
        dst.copy_(loaded_weight)

    def state_shape(self) -> tuple[int, int, int]:
        return self.num_heads, self.key_dim, self.value_dim

    def projection_sizes(self) -> list[int]:
        """Columns of the fused projection: q | k | v | b | a | gate."""
        return self.channel_sizes + [self.num_heads, self.num_heads, self.num_heads * self.value_dim]

    def forward(self, qkv, b, a, gate, run: int = 0) -> torch.Tensor:
        ctx = get_context()
        state = self.states[run]
        if state is None or ctx.state_slots is None:
            raise RuntimeError("the delta rule needs a bound state pool and a state slot per sequence")
        o = ops.gated_delta_rule(qkv, b, a, self.conv_weight.data, self.dt_bias.data, self.A_log.data, self.conv_inputs.pool(run), state, ctx.state_slots,
                                 ctx.cu_seqlens_q, ctx.context_lens, self.num_heads, self.qk_heads, self.key_dim, self.value_dim)
        return ops.group_rmsnorm_gate(o, self.norm.data, self.value_dim, self.eps, gate, "silu", gate_first=False)


class _StatePool(nn.Module):
    """A per-sequence fp32 state of fixed shape, one pool [slots, *shape] per pass (`states[run]`, bound by the runner)."""

    def __init__(self, shape: tuple, state_runs: int = 1):
        super().__init__()
        self._shape = tuple(int(n) for n in shape)
        self.state_runs = state_runs
        self.states: list = [None] * state_runs

    def state_shape(self) -> tuple:
        return self._shape

    def pool(self, run: int) -> torch.Tensor:
        ctx = get_context()
        if self.states[run] is None or ctx.state_slots is None:
            raise RuntimeError("a recurrent layer needs a bound state pool and a state slot per sequence")
        return self.states[run]


class DiagonalDecayRecurrence(_StatePool):
    """Per head a matrix memory S [dk, dv] in fp32 with a diagonal decay:

        S <- diag(w) S + (c k) v^T,      o = S^T q + d v

    w: one decay for each key channel, or a single one per head, c: a write strength per head (None: 1), d: a skip weight per head (None: 0),
    q and k possibly shared by groups of heads.  `read_first`: the token is read out before it is written and the state
    decayed, with a bonus u per head and key channel for the token itself, o = (S + diag(u) (c k) v^T)^T q + d v (the RWKV
    time mix).  The operands are fp32 (the mixers below make them from their projections);
    the scan walks this step's tokens of every sequence from the state its slot holds, or from zero when the sequence
    starts in this step (kernel: nvh_gated_linear_scan, csrc/linear_recurrence.hip)."""

    def __init__(self, num_heads: int, key_dim: int, value_dim: int, qk_groups: int | None = None, state_runs: int = 1):
        super().__init__((num_heads, value_dim, key_dim), state_runs)      # stored transposed: a column's key rows lie together
        self.num_heads, self.key_dim, self.value_dim, self.qk_groups = num_heads, key_dim, value_dim, qk_groups or num_heads

    def forward(self, q, k, w, v, run: int = 0, kscale=None, skip=None, read_first: bool = False, bonus=None) -> torch.Tensor:
        state = self.pool(run)
        ctx = get_context()
        return ops.gated_linear_scan(q, k, w, v, state, ctx.state_slots, ctx.cu_seqlens_q, ctx.context_lens, self.num_heads, self.key_dim,
                                     self.value_dim, self.qk_groups, kscale, skip, max_seqlen_q=ctx.max_seqlen_q or 0, read_first=read_first,
                                     bonus=bonus)


class HGRN2(nn.Module):
    """HGRN2 cell: a linear-attention memory without a key, the forget gate's complement taking its place.  Per head and key channel
    g = lower + (1 - lower) sigmoid(f + f_bias) in [lower, 1); S <- diag(g) S + (1 - g) v^T; o = S^T silu(q); q is the only
    other operand.  The read-out of a head is normalised (RMS along value_dim) by a single weight vector common to the heads.

    forward takes the column views q, f, v of the fused projection and returns [T, H * value_dim] in the activation type."""

    def __init__(self, num_heads: int, key_dim: int, value_dim: int, eps: float, state_runs: int = 1):
        super().__init__()
        n = num_heads * key_dim
        self.num_heads, self.key_dim, self.value_dim, self.eps = num_heads, key_dim, value_dim, eps
        self.f_bias = nn.Parameter(torch.zeros(n), requires_grad=False)
        self.lower = nn.Parameter(torch.zeros(n), requires_grad=False)
        self.norm = nn.Parameter(torch.ones(value_dim), requires_grad=False)
        self.memory = DiagonalDecayRecurrence(num_heads, key_dim, value_dim, state_runs=state_runs)

    def forward(self, q, f, v, run: int = 0) -> torch.Tensor:
        o = self.memory(*ops.hgrn2_prep(q, f, v, self.f_bias.data, self.lower.data), run)
        return ops.group_rmsnorm_gate(o, self.norm.data, self.value_dim, self.eps)


class GatedLinearAttention(nn.Module):
    """Gated linear attention: S <- diag(alpha) S + k v^T, o = S^T (q / sqrt(key_dim)), where every key channel has its own decay
    alpha = exp(log_sigmoid(z) / tau), z = W2 (low-rank input) + bias.  The read-out of a head is normalised (RMS along value_dim, a
    single weight vector common to the heads) and then gated by silu(gate).

    forward takes the column views q, k, v, gate and the low-rank decay input of the fused projection."""

    def __init__(self, num_heads: int, key_dim: int, value_dim: int, rank: int, tau: float, eps: float, state_runs: int = 1):
        super().__init__()
        self.num_heads, self.key_dim, self.value_dim, self.tau, self.eps = num_heads, key_dim, value_dim, float(tau), eps
        self.decay_up = MergedLinear(rank, [num_heads * key_dim], bias=True)          # W2 and its bias
        self.norm = nn.Parameter(torch.ones(value_dim), requires_grad=False)
        self.memory = DiagonalDecayRecurrence(num_heads, key_dim, value_dim, state_runs=state_runs)

    def forward(self, q, k, v, gate, lowrank, run: int = 0) -> torch.Tensor:
        z = self.decay_up(lowrank, out_f32=True)
        o = self.memory(*ops.gla_prep(q, k, v, z, self.key_dim ** -0.5, self.tau), run)
        return ops.group_rmsnorm_gate(o, self.norm.data, self.value_dim, self.eps, gate, "silu", gate_first=False)


class Mamba2(nn.Module):
    """The state-space-duality layer of Mamba-2.  The in-projection row holds z and x (inner = H * value_dim wide each), then B and C
    (groups * state_dim each), then one dt per head.  x, B, C pass a causal depthwise convolution (`taps` wide, last tap on the current token, continued
    across steps from the sequence's last taps - 1 inputs) and silu; dt = softplus(dt + dt_bias), unclamped.  Per head (B, C
    shared by the heads of a group):  S <- exp(-exp(A_log) dt) S + dt B x^T,  y = S^T C + D x,  S [N, value_dim] fp32.
    Read-out: y * silu(z), then an RMS norm taken separately over `norm_groups` equal slices, with a weight per column (gated, then normalised).

    forward takes the whole projection row and returns [T, inner] in the activation type."""

    def __init__(self, num_heads: int, value_dim: int, state_dim: int, groups: int, taps: int, norm_groups: int, eps: float, state_runs: int = 1):
        super().__init__()
        assert num_heads % groups == 0 and (num_heads * value_dim) % norm_groups == 0
        self.num_heads, self.value_dim, self.state_dim, self.groups, self.taps, self.norm_groups, self.eps = num_heads, value_dim, state_dim, groups, taps, norm_groups, eps
        self.inner, self.gn = num_heads * value_dim, groups * state_dim
        channels = self.inner + 2 * self.gn
        self.conv_weight = nn.Parameter(torch.zeros(channels, taps), requires_grad=False)
        self.conv_bias = nn.Parameter(torch.zeros(channels), requires_grad=False)
        self.dt_bias = nn.Parameter(torch.zeros(num_heads), requires_grad=False)
        self.A_log = nn.Parameter(torch.zeros(num_heads), requires_grad=False)
        self.D = nn.Parameter(torch.ones(num_heads, dtype=torch.float32), requires_grad=False)      # (an operand of the fp32 scan)
        self.norm = nn.Parameter(torch.ones(self.inner), requires_grad=False)
        self.conv_inputs = _StatePool((max(taps - 1, 1), channels), state_runs)     # the last taps - 1 inputs of x | B | C per sequence
        self.memory = DiagonalDecayRecurrence(num_heads, state_dim, value_dim, qk_groups=groups, state_runs=state_runs)

    def projection_sizes(self) -> list[int]:
        return [self.inner, self.inner + 2 * self.gn, self.num_heads]               # z | x B C | dt

    def forward(self, z, xbc, dt, run: int = 0) -> torch.Tensor:
        ctx = get_context()
        x, b, c, step, decay = ops.ssd_conv_prep(xbc, dt, self.conv_weight.data, self.conv_bias.data, self.dt_bias.data, self.A_log.data,
                                                 self.conv_inputs.pool(run), ctx.state_slots, ctx.cu_seqlens_q, ctx.context_lens,
                                                 self.num_heads, self.inner, self.gn)
        y = self.memory(c, b, decay, x, run, kscale=step, skip=self.D.data)
        return ops.group_rmsnorm_gate(y, self.norm.data, self.inner // self.norm_groups, self.eps, z, "silu", gate_first=True)


class Retention(nn.Module):
    """Retention: linear attention with one fixed decay per head and neither softmax nor denominator.  Per head, with rotary
    positions on the first `rot_dims` dimensions of q and k (frequencies given by the caller; pairs in halves unless
    `interleaved`) and k scaled by key_dim^(-1/2) after the rotation:

        S <- decay_h S + k v^T,      o = S^T q

    The read-out of a head is divided by its root mean square (no weight) and multiplied by silu(gate).

    forward takes the column views q, k, v, gate of the fused projection and returns [T, H * value_dim] in the activation type."""

    def __init__(self, num_heads: int, key_dim: int, value_dim: int, decays, eps: float, rot_dims: int = 0, freq: torch.Tensor | None = None,
                 mag: float = 1.0, interleaved: bool = False, state_runs: int = 1):
        super().__init__()
        decays = torch.as_tensor(decays, dtype=torch.float64).to(torch.float32)
        assert decays.numel() == num_heads and 0 <= rot_dims <= key_dim and rot_dims % 2 == 0
        self.num_heads, self.key_dim, self.value_dim, self.eps = num_heads, key_dim, value_dim, eps
        self.rot_dims, self.mag, self.interleaved = rot_dims, mag, interleaved
        dev = torch.empty(0).device
        self.register_buffer("decays", decays.to(dev), persistent=False)
        self.register_buffer("freq", None if freq is None else freq.to(dtype=torch.float32, device=dev), persistent=False)
        self.memory = DiagonalDecayRecurrence(num_heads, key_dim, value_dim, state_runs=state_runs)

    def forward(self, q, k, v, gate, positions, run: int = 0) -> torch.Tensor:
        oq, ok, ov = ops.rotary_qkv_prep(q, k, v, positions, self.freq, self.mag, self.rot_dims, self.interleaved, self.num_heads, self.key_dim,
                                         self.value_dim, 1.0, self.key_dim ** -0.5)
        w = self.decays.unsqueeze(0).expand(oq.shape[0], self.num_heads)      # one decay per head, the same for every token (row stride 0)
        o = self.memory(oq, ok, w, ov, run)
        return ops.group_rmsnorm_gate(o, None, self.value_dim, self.eps, gate, "silu", gate_first=False)


class TokenShift(_StatePool):
    """Blends every token's input with the input of the token before it, once per consumer: out[s] = h + (h_prev - h) mu[s].  The
    last input of a sequence is carried from step to step in its state slot (fp32 [1, width]; zeros before the first token)."""

    def __init__(self, width: int, consumers: int, state_runs: int = 1):
        super().__init__((1, width), state_runs)
        self.width, self.consumers = width, consumers
        self.mu = nn.Parameter(torch.zeros(consumers, width), requires_grad=False)

    def forward(self, h: torch.Tensor, run: int = 0) -> torch.Tensor:
        ctx = get_context()
        return ops.token_shift_mix(h, self.mu.data, self.pool(run), ctx.state_slots, ctx.cu_seqlens_q, ctx.context_lens)


class WKV(nn.Module):
    """The time mix of RWKV-6 ("Eagle and Finch: RWKV with Matrix-Valued States and Dynamic Recurrence", Peng et al.): per head a matrix
    memory S [dim, dim] in fp32 with a data-dependent decay per key channel, read BEFORE the token is written, the token itself
    entering its own read-out through a bonus u per head and channel:

        w = exp(-exp(W2 tanh(l) + w0)),      o = (S + diag(u) k v^T)^T r,      S <- diag(w) S + k v^T

    l: a low-rank projection of the (token-shifted) input.  The read-out of a head is divided by its root mean square, multiplied by a
    weight per column and by silu(gate).

    forward takes r, k, v, gate (projection outputs, each possibly of an input of its own) and the low-rank decay input l."""

    def __init__(self, num_heads: int, head_dim: int, rank: int, eps: float, state_runs: int = 1):
        super().__init__()
        n = num_heads * head_dim
        self.num_heads, self.head_dim, self.rank, self.eps = num_heads, head_dim, rank, eps
        self.w2 = nn.Parameter(torch.zeros(n, rank), requires_grad=False)
        self.w0 = nn.Parameter(torch.zeros(n), requires_grad=False)
        self.bonus = nn.Parameter(torch.zeros(num_heads, head_dim, dtype=torch.float32), requires_grad=False)      # (an operand of the fp32 scan)
        self.norm = nn.Parameter(torch.ones(n), requires_grad=False)
        self.memory = DiagonalDecayRecurrence(num_heads, head_dim, head_dim, state_runs=state_runs)

    def forward(self, r, k, v, gate, lowrank, run: int = 0) -> torch.Tensor:
        oq, ok, ow, ov = ops.wkv_prep(r, k, v, lowrank, self.w2.data, self.w0.data)
        o = self.memory(oq, ok, ow, ov, run, read_first=True, bonus=self.bonus.data)
        return ops.group_rmsnorm_gate(o, self.norm.data, self.head_dim, self.eps, gate, "silu", gate_first=False)


class StreamConv(_StatePool):
    """A short causal convolution of the fp32 residual stream over time, per column, added to the stream itself: what a sublayer reads
    is h_t = x_t + sum_k w[:, k] x_(t - taps + 1 + k) (no bias; the last tap lies on the token itself; zeros before the sequence's
    start).  The last taps - 1 rows of a sequence are carried from step to step in its state slot (fp32 [taps - 1, width])."""

    def __init__(self, width: int, taps: int, state_runs: int = 1):
        super().__init__((max(taps - 1, 1), width), state_runs)
        self.width, self.taps = width, taps
        self.weight = nn.Parameter(torch.zeros(width, taps), requires_grad=False)

    def forward(self, x: torch.Tensor, run: int = 0) -> torch.Tensor:
        """x fp32 [T, width] (left as it is) -> h in the activation type."""
        ctx = get_context()
        return ops.stream_conv(x, self.weight.data, self.pool(run), ctx.state_slots, ctx.cu_seqlens_q, ctx.context_lens)
