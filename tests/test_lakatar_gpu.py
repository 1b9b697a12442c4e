"""Lakatar through the engine against the plain float64 restatement in tests/lakatar_reference.py.

Every test makes its own small configuration and random weights (written as config.json + model.safetensors into a
temporary directory, so the config reader and the loader are part of what is tested), runs a schedule through
nanovllm.trace_replay.TraceReplay (the engine's runner, page/state manager and kernels) and compares logits - and, for
single layers, the residual stream - with the reference run over each whole sequence.  fp32 serving is compared
tightly, bf16 serving within the rounding of its products.
"""
import copy
import json
import math
import os

import numpy as np
import pytest
import torch

import lakatar_reference as R

pytestmark = pytest.mark.gpu

YARN = {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 2.0}
MOE_A = {"kind": "moe", "expert": {"ff": 24}, "router": {"experts": 6, "top": 2, "scale": 2.5, "groups": {"count": 3, "keep": 2}}, "shared": {"ff": 40}}
MOE_B = {"kind": "moe", "expert": {"ff": 36}, "router": {"experts": 7, "top": 3, "scale": 1.0, "groups": None}, "shared": None}
MOE_C = {"kind": "moe", "expert": {"ff": 16}, "router": {"experts": 8, "top": 4, "scale": 0.7, "groups": {"count": 4, "keep": 2}}, "shared": {"ff": 8}}
# key and value sizes that differ and that no tile divides, a rotation over part of the head
RET_A = {"type": "retention", "mlp": MOE_A,
         "mixer": {"heads": 3, "dim": 20, "vdim": 28, "decay": [0.9, 0.97, 0.995], "rot": {"base": 500.0, "dims": 12}}}
# heads of 32 / 16 (the scan's exact forms), the whole head rotated with scaled frequencies
RET_B = {"type": "retention", "mlp": None,
         "mixer": {"heads": 2, "dim": 32, "vdim": 16, "decay": [0.75, 0.999], "rot": {"base": 10000.0, "dims": 32, "scaling": YARN}}}
WKV_A = {"type": "wkv", "mixer": {"heads": 3, "dim": 20}, "mlp": MOE_B}
WKV_B = {"type": "wkv", "mixer": {"heads": 2, "dim": 32}, "mlp": None}
WKV_C = {"type": "wkv", "mixer": {"heads": 1, "dim": 6}, "mlp": MOE_C}
# cached row 40 + 8 = 48, value 40: the vector-ALU attention in both types
LAT_A = {"type": "latent_attention", "mlp": MOE_C,
         "mixer": {"heads": 3, "dim": 12, "rot_dim": 8, "vdim": 20, "q_rank": 24, "kv_rank": 40, "scale": 0.3, "rot": {"base": 700.0, "dims": 8}}}
# cached row 48 + 16 = 64, value 48: the matrix-core attention in bf16; scaled frequencies
LAT_B = {"type": "latent_attention", "mlp": None,
         "mixer": {"heads": 4, "dim": 16, "rot_dim": 16, "vdim": 24, "q_rank": 32, "kv_rank": 48, "scale": 0.2,
                   "rot": {"base": 10000.0, "dims": 16, "scaling": YARN}}}


def shared_latent(src_index, src, heads=2, dim=8, vdim=12, q_rank=16, scale=0.4, mlp=None):
    """A latent-attention layer that reads the latent of layer `src_index` (same kv_rank, rot_dim and rotation; all else its own)."""
    m = src["mixer"]
    return {"type": "latent_attention", "mlp": mlp,
            "mixer": {"heads": heads, "dim": dim, "rot_dim": m["rot_dim"], "vdim": vdim, "q_rank": q_rank, "kv_rank": m["kv_rank"], "scale": scale,
                      "rot": copy.deepcopy(m["rot"]), "kv_from": src_index}}


def config(layers, width=96, vocab=131, alpha=2.0, eps=1e-5):
    return {"architecture": "Lakatar", "vocab": vocab, "width": width, "norm": {"eps": eps}, "postln_alpha": alpha, "layers": copy.deepcopy(layers)}


CFG_MIX = config([WKV_A, LAT_A, RET_A, shared_latent(1, LAT_A, mlp=MOE_B), WKV_B])
CFG_FLAT = config([LAT_B, RET_B, shared_latent(0, LAT_B, heads=5, dim=16, vdim=16, q_rank=24), WKV_C], width=128, vocab=200, alpha=3.5, eps=1e-6)


def random_weights(cfg: dict, seed: int, ranks=(8, 5), calm: bool = False) -> dict:
    """bf16 weights in checkpoint naming; decays spread so that some channels forget fast and some hardly at all.  `calm`: router
    scores that vary little around corrections that lie far apart, so that the rounding of bf16 serving cannot flip a choice
    (the lively router, whose choice follows the token, is for fp32 serving)."""
    g = torch.Generator().manual_seed(seed)
    D, V = cfg["width"], cfg["vocab"]
    W = {}

    def mat(name, out, inp, scale=None):
        W[name] = torch.randn(out, inp, generator=g) * (scale if scale is not None else 1.0 / math.sqrt(inp))

    def vec(name, n, scale=1.0, shift=0.0):
        W[name] = shift + scale * torch.randn(n, generator=g)

    mat("embed", V, D, 1.0)
    mat("head", V, D)
    vec("final.norm", D, 0.2)
    n_wkv = 0
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        vec(p + "norm1", D, 0.2)
        vec(p + "ls1", D, 0.3, 1.0)
        h, d = m["heads"], m["dim"]
        if L["type"] == "retention":
            dv = m.get("vdim", d)
            for leaf, n in (("q", h * d), ("k", h * d), ("v", h * dv), ("g", h * dv)):
                mat(p + "mix." + leaf, n, D, 2.0 / math.sqrt(D))
            mat(p + "mix.o", D, h * dv)
        elif L["type"] == "wkv":
            n, rank = h * d, ranks[n_wkv % len(ranks)]
            n_wkv += 1
            for leaf in "rkvgw":
                W[p + "mix.mu." + leaf] = torch.rand(D, generator=g)
            for leaf in "rkvg":
                mat(p + "mix." + leaf, n, D, 2.0 / math.sqrt(D))
            mat(p + "mix.w1", rank, D)
            mat(p + "mix.w2", n, rank, 0.7)
            vec(p + "mix.w0", n, 1.5, -1.5)
            W[p + "mix.u"] = torch.randn(h, d, generator=g) * 0.5
            vec(p + "mix.norm", n, 0.2, 1.0)
            mat(p + "mix.o", D, n)
        else:
            dr, dv, rq, rkv = m["rot_dim"], m.get("vdim", d), m["q_rank"], m["kv_rank"]
            mat(p + "mix.dq", rq, D)
            vec(p + "mix.dq.norm", rq, 0.2, 1.0)
            mat(p + "mix.uq", h * (d + dr), rq, 2.0 / math.sqrt(rq))
            if m.get("kv_from") is None:
                mat(p + "mix.dkv", rkv + dr, D)
                vec(p + "mix.dkv.norm", rkv, 0.2, 1.0)
            mat(p + "mix.uk", h * d, rkv, 2.0 / math.sqrt(rkv))
            mat(p + "mix.uv", h * dv, rkv)
            mat(p + "mix.g", h, D)
            mat(p + "mix.o", D, h * dv)
        mlp = L.get("mlp")
        if not mlp:
            continue
        vec(p + "norm2", D, 0.2)
        vec(p + "ls2", D, 0.3, 1.0)
        E, ff = mlp["router"]["experts"], mlp["expert"]["ff"]
        for e in range(E):
            mat(f"{p}mlp.e{e}.gate", ff, D)
            mat(f"{p}mlp.e{e}.up", ff, D)
            mat(f"{p}mlp.e{e}.down", D, ff)
        if calm:
            mat(p + "mlp.router", E, D, 0.2 / math.sqrt(D))
            W[p + "mlp.correction"] = torch.linspace(-0.6, 0.6, E)[torch.randperm(E, generator=g)]
        else:
            mat(p + "mlp.router", E, D, 3.0 / math.sqrt(D))
            vec(p + "mlp.correction", E, 0.15)                   # (some negative: a masked group must count as minus infinity, not 0)
        if mlp.get("shared"):
            mat(p + "mlp.shared.gate", mlp["shared"]["ff"], D)
            mat(p + "mlp.shared.up", mlp["shared"]["ff"], D)
            mat(p + "mlp.shared.down", D, mlp["shared"]["ff"])
            mat(p + "mlp.shared.sg", 1, D, 2.0 / math.sqrt(D))
    return {k: v.to(torch.bfloat16) for k, v in W.items()}


def write_model(path, cfg: dict, weights: dict) -> str:
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in weights.items()}, os.path.join(path, "model.safetensors"))
    return str(path)


class Case:
    """A model on disk, its reference weights and cached reference logits per token list."""

    def __init__(self, tmp, cfg, seed=0, weights=None, calm=False):
        self.cfg = cfg
        w = weights if weights is not None else random_weights(cfg, seed, calm=calm)
        self.path = write_model(tmp, cfg, w)
        self.W = {k: v.double() for k, v in w.items()}
        self._ref = {}

    def ref(self, tokens):
        key = tuple(tokens)
        if key not in self._ref:
            self._ref[key] = R.forward(self.W, self.cfg, list(tokens)).numpy()
        return self._ref[key]

    def replay(self, dtype="float32", max_tokens=2048, slots=4):
        from nanovllm.trace_replay import TraceReplay
        return TraceReplay(self.path, dtype, max_tokens, slots)


def tokens_of(cfg, n, seed):
    return torch.randint(0, cfg["vocab"], (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def rel_err(got, want):
    """Largest row error, mean removed, relative to the spread of the reference logits."""
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    return float(np.sqrt((d ** 2).mean(-1)).max() / want.std())


TOL = {"float32": 2e-4, "bfloat16": 6e-2}


@pytest.fixture(scope="module")
def mix_case(tmp_path_factory):
    return Case(tmp_path_factory.mktemp("lakatar_mix"), CFG_MIX, seed=1)


@pytest.fixture(scope="module")
def mix_case_calm(tmp_path_factory):
    return Case(tmp_path_factory.mktemp("lakatar_mix_calm"), CFG_MIX, seed=1, calm=True)


@pytest.fixture(scope="module")
def flat_case(tmp_path_factory):
    return Case(tmp_path_factory.mktemp("lakatar_flat"), CFG_FLAT, seed=2, calm=True)


def case_for(dtype, lively, calm):
    return calm if dtype == "bfloat16" else lively


def run_schedule(rp, case, requests: dict, schedule: list, dtype: str, tol=None):
    """schedule: list of steps, each a list of (request id, token count); every position's logits are asked for and
    compared with the reference of the whole request.  Requests end when their tokens are used up."""
    at = {r: 0 for r in requests}
    worst = 0.0
    for step in schedule:
        entries, spans, end = [], [], []
        for rid, count in step:
            lo, hi = at[rid], at[rid] + count
            entries.append({"id": rid, "tokens": requests[rid][lo:hi], "want": list(range(count))})
            spans.append((rid, lo, hi))
            at[rid] = hi
            if hi == len(requests[rid]):
                end.append(rid)
        got = rp.step(entries, end)
        row = 0
        for rid, lo, hi in spans:
            want = case.ref(requests[rid])[lo:hi]
            err = rel_err(got[row:row + hi - lo], want)
            assert err < (tol or TOL[dtype]), f"request {rid} tokens {lo}..{hi}: error {err:.3g}"
            worst = max(worst, err)
            row += hi - lo
    assert all(at[r] == len(requests[r]) for r in requests)
    return worst


# ----------------------------------------------------------------------------------------------------- single mechanisms
@pytest.mark.parametrize("layer", [RET_A, RET_B, WKV_A, WKV_B, WKV_C, LAT_A, LAT_B],
                         ids=["retention(ragged, part rotated)+moe(groups)", "retention(exact, scaled rotary)", "wkv(ragged)+moe(no groups)", "wkv(exact)",
                              "wkv(one small head)+moe", "latent(vector ALU)+moe", "latent(matrix cores in bf16, scaled rotary)"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_one_layer_stream_matches(tmp_path, layer, dtype):
    """One layer of each kind: the residual stream after it and the logits."""
    cfg = config([layer], width=72, vocab=50, alpha=1.5)
    case = Case(tmp_path, cfg, seed=3, calm=dtype == "bfloat16")
    toks = tokens_of(cfg, 70, 5)
    rp = case.replay(dtype)
    try:
        rp.runner.model.collect = []
        got = rp.step([{"id": 0, "tokens": toks, "want": list(range(len(toks)))}], [0])
        stream = rp.runner.model.collect[0].cpu().numpy()
    finally:
        rp.close()
    col = []
    want = R.forward(case.W, cfg, toks, col).numpy()
    assert np.abs(stream - col[0].numpy()).max() < (1e-4 if dtype == "float32" else 0.15) * max(1.0, float(col[0].abs().max()))
    assert rel_err(got, want) < TOL[dtype]


def test_every_layer_of_a_stack_with_a_shared_latent(mix_case):
    """Five layers, the fourth reading the latent the second cached: the stream after every layer."""
    toks = tokens_of(CFG_MIX, 40, 7)
    rp = mix_case.replay("float32")
    try:
        rp.runner.model.collect = []
        rp.step([{"id": 0, "tokens": toks, "want": [0]}], [0])
        streams = [c.cpu().numpy() for c in rp.runner.model.collect]
    finally:
        rp.close()
    col = []
    R.forward(mix_case.W, CFG_MIX, toks, col)
    assert len(streams) == len(col) == 5
    for n, (a, b) in enumerate(zip(streams, col)):
        assert np.abs(a - b.numpy()).max() < 2e-4 * max(1.0, float(b.abs().max())), f"layer {n}"


def test_scan_that_reads_before_it_writes():
    """The diagonal-decay scan in its read-first form with a bonus for the token itself, against the recurrence written out: key
    sizes that are and are not multiples of 16 and of 4; one sequence continued from a state, one fresh, slots out of order;
    portions long enough to be walked in segments beside short ones."""
    from nanovllm import ops
    g = torch.Generator().manual_seed(0)
    for H, dk, dv, lens in [(3, 20, 20, [9, 5]), (2, 16, 48, [9, 5]), (2, 48, 48, [9, 5]), (1, 37, 5, [9, 5]), (1, 128, 64, [9, 5]), (1, 6, 6, [9, 5]),
                            (2, 32, 24, [300, 7]), (1, 64, 16, [1, 555]), (2, 16, 8, [256, 257]), (1, 48, 48, [513, 2])]:
        past = [4, 0]
        T = sum(lens)
        q, k = torch.randn(T, H * dk, generator=g), torch.randn(T, H * dk, generator=g)
        w = torch.rand(T, H * dk, generator=g) ** (0.02 if max(lens) > 100 else 1.0)       # (long runs: decays near one, so far tokens count)
        v = torch.randn(T, H * dv, generator=g)
        u = torch.randn(H, dk, generator=g)
        state = torch.randn(5, H, dk, dv, generator=g)
        slots = [3, 1]
        want, new_state = torch.zeros(T, H * dv, dtype=torch.float64), state.double().clone()
        t0 = 0
        for b, n in enumerate(lens):
            for h in range(H):
                S = state[slots[b], h].double() if past[b] else torch.zeros(dk, dv, dtype=torch.float64)
                ks, vs = slice(h * dk, (h + 1) * dk), slice(h * dv, (h + 1) * dv)
                for t in range(t0, t0 + n):
                    kv = torch.outer(k[t, ks].double(), v[t, vs].double())
                    want[t, vs] = (S + u[h].double()[:, None] * kv).T @ q[t, ks].double()
                    S = w[t, ks].double()[:, None] * S + kv
                new_state[slots[b], h] = S
            t0 += n
        st = state.transpose(2, 3).contiguous().cuda()          # the pool holds S transposed: [slots, H, dv, dk]
        cu = torch.tensor([0, lens[0], T], dtype=torch.int32).cuda()
        ctx = torch.tensor([lens[0] + past[0], lens[1] + past[1]], dtype=torch.int32).cuda()
        got = ops.gated_linear_scan(q.cuda(), k.cuda(), w.cuda(), v.cuda(), st, torch.tensor(slots, dtype=torch.int32).cuda(), cu, ctx, H, dk, dv,
                                    max_seqlen_q=max(lens), read_first=True, bonus=u.cuda())
        assert (got.cpu().double() - want).abs().max() < 1e-4 * max(1.0, float(want.abs().max())), (H, dk, dv, lens)
        assert (st.cpu().double().transpose(2, 3) - new_state).abs().max() < 1e-4 * max(1.0, float(new_state.abs().max()))


def test_router_by_scores_with_correction_groups_and_scale():
    """Scores, choice and weights of the score router against the formulas: corrections that change the choice but not the weights,
    groups whose best choice score decides (negative choice scores included), every expert eligible when all groups are kept,
    more rows over the same input (the shared expert's gate)."""
    from nanovllm import ops
    g = torch.Generator().manual_seed(1)
    for E, top, groups, keep, scale in [(6, 2, 3, 2, 2.5), (7, 3, 1, 1, 1.0), (8, 4, 4, 2, 0.7), (64, 6, 8, 3, 1.0), (130, 8, 10, 4, 1.5), (3, 3, 3, 3, 1.0),
                                        (12, 2, 4, 1, 1.0), (1, 1, 1, 1, 2.0), (300, 5, 10, 3, 1.0)]:
        x, w = torch.randn(33, 70, generator=g), torch.randn(E, 70, generator=g) * 0.3
        corr = torch.randn(E, generator=g) * 0.2 - 0.3          # mostly negative: zeros in place of minus infinity would win
        aux = torch.randn(2, 70, generator=g)
        for cast in (torch.float32, torch.bfloat16):
            xa, wa, ca, aa = x.to(cast), w.to(cast), corr.to(cast), aux.to(cast)
            s = torch.softmax(xa.double() @ wa.double().T, -1)
            choice = s + ca.double()
            if groups > 1:
                per = E // groups
                best = choice.view(-1, groups, per).max(-1).values.topk(keep, -1).indices
                ok = torch.zeros(33, groups, dtype=torch.bool).scatter_(1, best, True).repeat_interleave(per, 1)
                choice = choice.masked_fill(~ok, -math.inf)
            idx = choice.topk(top, -1).indices
            ids, wts, gate, scores = ops.moe_route_scored(xa.cuda(), wa.cuda(), top, ca.cuda(), groups, keep, scale, aux=aa.cuda(), want_scores=True)
            assert (scores.cpu().double() - s).abs().max() < 1e-5
            assert torch.equal(ids.cpu().long(), idx), (E, top, groups, keep)
            assert (wts.cpu().double() - s.gather(1, idx) * scale).abs().max() < 1e-5
            assert (gate.cpu().double() - xa.double() @ aa.double().T).abs().max() < 1e-4
    # no correction, no further rows; a tie goes to the lower expert
    x = torch.zeros(1, 8)
    ids, wts, gate = ops.moe_route_scored(x.cuda(), torch.randn(4, 8, generator=g).cuda(), 2)
    assert ids.cpu().tolist() == [[0, 1]] and gate is None and (wts.cpu() - 0.25).abs().max() < 1e-6


def test_gated_shared_expert_in_the_combine():
    from nanovllm import ops
    g = torch.Generator().manual_seed(2)
    T, E, top, N = 40, 5, 2, 52
    ids = torch.randint(0, E, (T, top), generator=g).int()
    wts, gate = torch.rand(T, top, generator=g), torch.randn(T, 1, generator=g)
    y, shared = torch.randn(T * top, N, generator=g), torch.randn(T, N, generator=g)
    plan = ops.moe_align(ids.cuda(), E)
    pos = plan["pos_of_pair"].cpu().view(T, top).long()
    out = ops.moe_combine(y.cuda(), plan, wts.cuda(), shared.cuda(), gate.cuda()).cpu()
    want = (wts[:, :, None] * y[pos]).sum(1) + torch.sigmoid(gate) * shared
    assert (out - want).abs().max() < 1e-5


def test_sum_then_norm_kernel_against_its_formula():
    from nanovllm import ops
    g = torch.Generator().manual_seed(3)
    unit = lambda v: v / torch.sqrt((v * v).mean(-1, keepdim=True) + 1e-5)
    for dim in (50, 96, 1000):
        x, y, y32 = (torch.randn(9, dim, generator=g) for _ in range(3))
        ls, w = torch.randn(dim, generator=g), torch.randn(dim, generator=g) * 0.3
        xg = x.cuda()
        h = ops.residual_postnorm(xg, w.cuda(), 1e-5, y=y.cuda(), y32=y32.cuda(), layer_scale=ls.cuda(), alpha=2.5, weight_offset=1.0)
        want = unit(2.5 * x + ls * (y + y32)) * (1 + w)
        assert (xg.cpu() - want).abs().max() < 1e-5 and (h.cpu() - want).abs().max() < 1e-5
        xg = x.cuda()
        h = ops.residual_postnorm(xg, w.cuda(), 1e-5, y=y.cuda())                  # no scale, alpha 1, a plain weight
        assert (h.cpu() - unit(x + y) * w).abs().max() < 1e-5
        xg = x.cuda()
        h = ops.residual_postnorm(xg, w.cuda(), 1e-5, weight_offset=1.0, in_place=False)       # the norm alone, the stream untouched
        assert torch.equal(xg.cpu(), x) and (h.cpu() - unit(x) * (1 + w)).abs().max() < 1e-5
        hb = ops.residual_postnorm(x.cuda(), w.bfloat16().cuda(), 1e-5, y=y.bfloat16().cuda(), weight_offset=1.0)
        assert hb.dtype == torch.bfloat16 and (hb.float().cpu() - unit(x + y.bfloat16().float()) * (1 + w.bfloat16().float())).abs().max() < 0.05


def test_token_shift_takes_the_previous_token_from_the_step_or_the_slot():
    from nanovllm import ops
    g = torch.Generator().manual_seed(4)
    dim, n = 37, 3
    h, mu = torch.randn(8, dim, generator=g), torch.rand(n, dim, generator=g)
    state = torch.randn(4, 1, dim, generator=g)
    # sequence 0: 5 tokens continued (slot 2 holds its last input); sequence 1: 3 tokens, fresh, in slot 0
    st = state.clone().cuda()
    cu, ctx = torch.tensor([0, 5, 8], dtype=torch.int32).cuda(), torch.tensor([9, 3], dtype=torch.int32).cuda()
    out = ops.token_shift_mix(h.cuda(), mu.cuda(), st, torch.tensor([2, 0], dtype=torch.int32).cuda(), cu, ctx).cpu()
    prev = torch.cat([state[2], h[:4], torch.zeros(1, dim), h[5:7]])
    for s in range(n):
        assert (out[s] - (h + (prev - h) * mu[s])).abs().max() < 1e-6
    assert torch.equal(st.cpu()[2, 0], h[4]) and torch.equal(st.cpu()[0, 0], h[7]) and torch.equal(st.cpu()[1], state[1])
    # one token per sequence, no offsets (the shape of a captured decode step); a padded row (slot -1) is left alone
    st = state.clone().cuda()
    out = ops.token_shift_mix(h[:3].cuda(), mu.cuda(), st, torch.tensor([1, -1, 3], dtype=torch.int32).cuda(), None, torch.tensor([5, 0, 1], dtype=torch.int32).cuda()).cpu()
    assert (out[1][0] - (h[0] + (state[1, 0] - h[0]) * mu[1])).abs().max() < 1e-6 and (out[1][2] - (h[2] - h[2] * mu[1])).abs().max() < 1e-6
    assert torch.equal(st.cpu()[1, 0], h[0]) and torch.equal(st.cpu()[3, 0], h[2]) and torch.equal(st.cpu()[0], state[0])


def test_products_per_head():
    """y[t, h] = x[t, h] W[h]^T with heads at a stride in the input row and at another in the output row, both types, ragged sizes."""
    from nanovllm import ops
    g = torch.Generator().manual_seed(5)
    for T, H, N, K, xs, ys in [(70, 3, 40, 12, 20, 48), (5, 4, 16, 64, 64, 16), (130, 2, 100, 72, 80, 100)]:
        x, w = torch.randn(T, (H - 1) * xs + K + 3, generator=g), torch.randn(H, N, K, generator=g)
        for cast, tol in ((torch.float32, 1e-4), (torch.bfloat16, 3e-2)):
            xa, wa = x.to(cast), w.to(cast)
            out = torch.zeros(T, (H - 1) * ys + N + 2, dtype=cast).cuda()
            ops.linear_heads(xa.cuda(), wa.cuda(), xs, out=out, out_head_stride=ys)
            for h in range(H):
                want = xa[:, h * xs:h * xs + K].double() @ wa[h].double().T
                assert (out.cpu()[:, h * ys:h * ys + N].double() - want).abs().max() < tol * max(1.0, float(want.abs().max()))
            assert float(out.cpu()[:, -2:].abs().max()) == 0.0           # nothing is written beyond a head's N columns


# ----------------------------------------------------------------------------------------------------- schedules
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prefill_then_token_by_token(mix_case, mix_case_calm, dtype):
    mix_case = case_for(dtype, mix_case, mix_case_calm)
    toks = tokens_of(CFG_MIX, 90, 11)
    rp = mix_case.replay(dtype)
    try:
        run_schedule(rp, mix_case, {"a": toks}, [[("a", 50)]] + [[("a", 1)]] * 40, dtype)
        # the first tokens of a sequence, one by one from the very start (no previous token to shift in, empty memories, one key)
        run_schedule(rp, mix_case, {"b": toks[:20]}, [[("b", 1)]] * 20, dtype)
    finally:
        rp.close()


def test_portions_of_every_size_give_the_same_logits(mix_case):
    toks = tokens_of(CFG_MIX, 120, 13)
    rp = mix_case.replay("float32")
    try:
        for sizes in ([120], [2] * 60, [3, 2, 17, 2, 33, 16, 2, 45], [64, 56], [1, 119]):
            assert sum(sizes) == 120
            run_schedule(rp, mix_case, {"a": toks}, [[("a", s)] for s in sizes], "float32")
    finally:
        rp.close()


def test_cutting_does_not_change_a_bit_of_the_recurrent_path(tmp_path):
    """Recurrent mixers only (no attention, whose key tiles see the cut): one piece, portions and single tokens give identical
    logits, the shifted-in previous token included."""
    cfg = config([WKV_A, RET_A, WKV_B, RET_B], width=64, vocab=64)
    case = Case(tmp_path, cfg, seed=5)
    toks = tokens_of(cfg, 48, 2)
    rp = case.replay("float32")
    try:
        whole = rp.step([{"id": 0, "tokens": toks, "want": [47]}], [0])
        rp.step([{"id": 1, "tokens": toks[:20], "want": []}])
        rp.step([{"id": 1, "tokens": toks[20:41], "want": []}])
        for p in range(41, 47):
            rp.step([{"id": 1, "tokens": toks[p:p + 1], "want": []}])
        cut = rp.step([{"id": 1, "tokens": toks[47:], "want": [0]}], [1])
    finally:
        rp.close()
    assert np.array_equal(whole, cut)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mixed_batches_of_unequal_requests(mix_case, mix_case_calm, dtype):
    mix_case = case_for(dtype, mix_case, mix_case_calm)
    reqs = {"a": tokens_of(CFG_MIX, 75, 21), "b": tokens_of(CFG_MIX, 9, 22), "c": tokens_of(CFG_MIX, 33, 23), "d": tokens_of(CFG_MIX, 2, 24)}
    sched = [[("a", 30), ("b", 3)], [("a", 1), ("b", 2), ("c", 20)], [("b", 1), ("a", 17), ("c", 1), ("d", 2)], [("c", 2), ("a", 27), ("b", 3)],
             [("c", 10)]]
    rp = mix_case.replay(dtype)
    try:
        run_schedule(rp, mix_case, reqs, sched, dtype)
    finally:
        rp.close()


def test_pages_and_slots_are_used_again(flat_case):
    """A pool of three pages and two state slots serves six requests one after another and in pairs: every request after
    the first two runs on pages and slots (memories, shifted-in tokens) that others have left behind."""
    reqs = {i: tokens_of(CFG_FLAT, n, 30 + i) for i, n in enumerate([300, 120, 257, 40, 256, 130])}
    rp = flat_case.replay("float32", max_tokens=256, slots=2)            # ceil(256/256) + 2 = 3 pages
    assert len(rp.scheduler.block_manager.blocks) == 3 and rp.scheduler.block_manager.num_state_slots == 2
    try:
        run_schedule(rp, flat_case, {0: reqs[0]}, [[(0, 200)], [(0, 100)]], "float32")
        run_schedule(rp, flat_case, {1: reqs[1], 2: reqs[2]}, [[(1, 100), (2, 7)], [(1, 20), (2, 250)]], "float32")
        run_schedule(rp, flat_case, {3: reqs[3], 4: reqs[4]}, [[(4, 255), (3, 39)], [(3, 1), (4, 1)]], "float32")
        run_schedule(rp, flat_case, {5: reqs[5]}, [[(5, 129)], [(5, 1)]], "float32")
        assert len(rp.scheduler.block_manager.free_block_ids) == 3 and len(rp.scheduler.block_manager.free_state_slots) == 2
    finally:
        rp.close()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_page_borders_and_segment_sizes_in_prompts_and_in_decoding(flat_case, dtype):
    """Portions that end one token before, at and after a page border, then decoding across the next one; portions of 255, 256 and
    257 tokens (from 256 on the recurrent layers walk a portion in segments) and of 511, 512, 513."""
    toks = tokens_of(CFG_FLAT, 530, 41)
    rp = flat_case.replay(dtype, max_tokens=1100)
    try:
        run_schedule(rp, flat_case, {"a": toks}, [[("a", 255)], [("a", 1)], [("a", 1)], [("a", 2)], [("a", 251)], [("a", 3)]] + [[("a", 1)]] * 17, dtype)
        for first in (256, 257, 511, 512, 513):
            run_schedule(rp, flat_case, {"b": toks[:first + 8]}, [[("b", first)], [("b", 7)], [("b", 1)]], dtype)
    finally:
        rp.close()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_one_token_steps_of_sequences_of_unequal_length(flat_case, dtype):
    """Steps in which every sequence brings one token (the form in which the heads that share a latent share a workgroup and, in
    bf16, a sequence's 64-key tiles are dealt out to several workgroups and merged): contexts of one to five tiles side by side, so
    that most workgroups of the short ones find no tile; then fewer sequences as the short requests end."""
    reqs = {i: tokens_of(CFG_FLAT, n, 80 + i) for i, n in enumerate([36, 75, 135, 300])}
    first = {0: 30, 1: 64, 2: 129, 3: 290}
    sched = [[(i, first[i]) for i in reqs]] + [[(i, 1) for i in reqs if first[i] + k < len(reqs[i])] for k in range(11)]
    rp = flat_case.replay(dtype, max_tokens=1100)
    try:
        run_schedule(rp, flat_case, reqs, [st for st in sched if st], dtype)
    finally:
        rp.close()


def test_long_decoding(mix_case):
    toks = tokens_of(CFG_MIX, 230, 43)
    rp = mix_case.replay("float32", max_tokens=512)
    try:
        run_schedule(rp, mix_case, {"a": toks}, [[("a", 5)]] + [[("a", 1)]] * 225, "float32")
    finally:
        rp.close()


# ----------------------------------------------------------------------------------------------------- faults that random weights would hide
def sharp_latent_case(tmp, shared: bool):
    """Latent attention whose unrotated keys equal its unrotated queries (the two latents and their expansions share weights), with
    no weight on the rotated part and a large scale: a query puts nearly all its weight on the earlier occurrence of its own token.
    `shared`: a first layer that is switched off (zero layer scale) owns the latent, the second reads it."""
    own = {"type": "latent_attention", "mlp": None,
           "mixer": {"heads": 2, "dim": 32, "rot_dim": 16, "vdim": 32, "q_rank": 48, "kv_rank": 48, "scale": 0.5, "rot": {"base": 10000.0, "dims": 16}}}
    layers = [own, shared_latent(0, own, heads=2, dim=32, vdim=32, q_rank=48, scale=0.5)] if shared else [own]
    cfg = config(layers, width=64, vocab=900, alpha=1.0)
    w = random_weights(cfg, 9)
    last = len(layers) - 1
    p = f"l{last}.mix."
    w[p + "dq"] = w["l0.mix.dkv"][:48].clone()
    w[p + "dq.norm"] = w["l0.mix.dkv.norm"].clone()
    uq = w[p + "uq"].view(2, 48, 48).clone()
    uq[:, :32] = w[p + "uk"].view(2, 32, 48)
    uq[:, 32:] = 0
    w[p + "uq"] = uq.view(96, 48)
    w[p + "uv"] = w[p + "uv"] * 4
    if shared:
        w["l0.ls1"] = torch.zeros_like(w["l0.ls1"])            # the owner adds nothing: layer 1 sees the normed embeddings, as its latent does
        w["l0.norm1"] = torch.zeros_like(w["l0.norm1"])
    return Case(tmp, cfg, weights=w), cfg


@pytest.mark.parametrize("shared", [False, True], ids=["own latent", "latent of an earlier layer"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_far_key_decides_wherever_it_lies(tmp_path, dtype, shared):
    """The last token repeats an earlier one, which then gets nearly all the weight among 600 keys: at the start, around both page
    borders, right before the query.  Whole prompt in one step, and the last token decoded alone."""
    case, cfg = sharp_latent_case(tmp_path, shared)
    n = 600
    base = list(range(1, n + 1))
    rp = case.replay(dtype, max_tokens=1300)
    try:
        for far in (0, 3, 255, 256, 257, 511, 512, n - 2):
            toks = base[:n - 1] + [base[far]]
            ref = case.ref(toks)[-1:]
            assert rel_err(case.ref(base[:n - 1] + [899])[-1:], ref) > 0.3, far       # the key matters: without it the logits are others
            whole = rp.step([{"id": 0, "tokens": toks, "want": [n - 1]}], [0])
            rp.step([{"id": 1, "tokens": toks[:n - 1], "want": []}])
            decoded = rp.step([{"id": 1, "tokens": toks[n - 1:], "want": [0]}], [1])
            tol = TOL[dtype] if dtype == "float32" else 0.15      # (sharp weights magnify the rounding of bf16 scores)
            assert rel_err(whole, ref) < tol and rel_err(decoded, ref) < tol, far
    finally:
        rp.close()


def test_recurrent_memories_carry_a_token_from_far_back(tmp_path):
    """Decays near one keep a memory for hundreds of tokens: the first token still shapes the last logits in both recurrent mixers,
    and a state that were lost or reset between portions would show."""
    ret = {"type": "retention", "mlp": None, "mixer": {"heads": 2, "dim": 16, "vdim": 16, "decay": [0.999, 0.9995], "rot": {"base": 100.0, "dims": 8}}}
    for kind, layer in (("retention", ret), ("wkv", WKV_B)):
        cfg = config([layer], width=48, vocab=90, alpha=1.0)
        w = random_weights(cfg, 4)
        if kind == "wkv":
            w["l0.mix.w0"] = torch.full_like(w["l0.mix.w0"], -6.5)
            w["l0.mix.w2"] = w["l0.mix.w2"] * 0.1
        case = Case(tmp_path / kind, cfg, weights=w)
        toks = tokens_of(cfg, 400, 8)
        changed = [(toks[0] + 1) % 90] + toks[1:]
        assert rel_err(case.ref(changed)[-1:], case.ref(toks)[-1:]) > 5 * TOL["float32"], kind      # 400 tokens later it still shows
        rp = case.replay("float32", max_tokens=1024)
        try:
            run_schedule(rp, case, {"a": toks}, [[("a", 100)], [("a", 156)], [("a", 1)], [("a", 140)], [("a", 2)], [("a", 1)]], "float32")
            # portions long enough to be scanned in segments, beside a short request; then the state they left is decoded from
            run_schedule(rp, case, {"b": toks, "c": toks[:9]}, [[("b", 290), ("c", 8)], [("b", 109), ("c", 1)], [("b", 1)]], "float32")
        finally:
            rp.close()


def test_the_bonus_and_the_shift_show(tmp_path):
    """With a zero bonus or without the shifted-in token the reference itself changes clearly, so the agreement of the other
    tests is not one that a missing bonus or shift could share."""
    cfg = config([WKV_B], width=48, vocab=90, alpha=1.0)
    case = Case(tmp_path, cfg, seed=4)
    toks = tokens_of(cfg, 30, 1)
    full = case.ref(toks)
    for leaf in ("u", "mu.k"):
        W = dict(case.W)
        W["l0.mix." + leaf] = torch.zeros_like(W["l0.mix." + leaf])
        assert rel_err(R.forward(W, cfg, toks).numpy(), full) > 0.05, leaf


# ----------------------------------------------------------------------------------------------------- other sizes
def test_sizes_no_kernel_tile_divides(tmp_path):
    """A width that is no multiple of 8; one expert of which one is taken; every group kept; twenty query heads over one latent (more
    than a one-token step shares a workgroup among); a latent of 300 (wider than 256 value columns), a two-wide rotated part; heads of 72 and 130 in the
    recurrent layers; a first layer that reads a latent no layer has yet filled is refused."""
    layers = [{"type": "latent_attention", "mlp": {"kind": "moe", "expert": {"ff": 10}, "router": {"experts": 1, "top": 1, "scale": 1.0, "groups": {"count": 1, "keep": 1}}, "shared": {"ff": 6}},
               "mixer": {"heads": 20, "dim": 4, "rot_dim": 16, "vdim": 4, "q_rank": 10, "kv_rank": 32, "scale": 0.5, "rot": {"base": 50.0, "dims": 16}}},
              {"type": "wkv", "mixer": {"heads": 1, "dim": 130}, "mlp": {"kind": "moe", "expert": {"ff": 12}, "router": {"experts": 4, "top": 2, "scale": 1.0, "groups": {"count": 2, "keep": 2}}, "shared": None}},
              {"type": "latent_attention", "mlp": None,
               "mixer": {"heads": 1, "dim": 50, "rot_dim": 2, "vdim": 70, "q_rank": 7, "kv_rank": 300, "scale": 0.1, "rot": {"base": 10.0, "dims": 2}}},
              {"type": "retention", "mlp": None, "mixer": {"heads": 1, "dim": 72, "vdim": 10, "decay": [0.5], "rot": {"base": 3.0, "dims": 72}}},
              {"type": "latent_attention", "mlp": None,
               "mixer": {"heads": 20, "dim": 8, "rot_dim": 16, "vdim": 8, "q_rank": 12, "kv_rank": 32, "scale": 0.5, "rot": {"base": 50.0, "dims": 16}, "kv_from": 0}}]
    cfg = config(layers, width=50, vocab=37, alpha=1.0)
    case = Case(tmp_path, cfg, weights=random_weights(cfg, 6, ranks=(3,), calm=True))
    toks = tokens_of(cfg, 80, 3)
    for dtype in ("float32", "bfloat16"):
        rp = case.replay(dtype)
        try:
            run_schedule(rp, case, {"a": toks, "b": toks[:7]}, [[("a", 33), ("b", 5)], [("a", 1), ("b", 2)], [("a", 44)], [("a", 1)], [("a", 1)]], dtype,
                         tol=None if dtype == "float32" else 0.15)     # (50 columns wide and five layers deep: the rounding of bf16 adds up layer by layer)
        finally:
            rp.close()
    bad = config([shared_latent(1, LAT_A), LAT_A], width=50, vocab=37)
    with pytest.raises(ValueError):
        from nanovllm.models.lakatar import LakatarForCausalLM
        from types import SimpleNamespace
        LakatarForCausalLM(SimpleNamespace(**bad))


# ----------------------------------------------------------------------------------------------------- the engine's own entry point
def test_greedy_generation_through_the_engine(mix_case):
    """LLM.generate with temperature 0 (scheduler, chunked prefill, captured graphs, sampling kernel) against greedy decoding of
    the reference."""
    from nanovllm import LLM, SamplingParams
    prompts = [tokens_of(CFG_MIX, n, 50 + n) for n in (5, 40, 17)]
    llm = LLM(mix_case.path, dtype="float32", max_num_seqs=4, max_num_batched_tokens=32, max_model_len=128, num_kvcache_blocks=6,
              chunked_prefill=True)
    try:
        assert llm.model_runner.graphs, "one-token steps are expected to replay captured graphs"
        outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True), use_tqdm=False)
    finally:
        llm.exit()
    for prompt, out in zip(prompts, outs):
        toks = list(prompt)
        for _ in range(12):
            toks.append(int(R.forward(mix_case.W, CFG_MIX, toks)[-1].argmax()))
        assert out["token_ids"] == toks[len(prompt):]


def test_captured_decode_steps_match_eager_ones(flat_case):
    """One-token steps replayed from the captured graph (routing, expert tiles, states and the shared latent inside it) against the
    same steps run eagerly: several replays, with eager work between them."""
    from nanovllm.config import Config
    from nanovllm.engine.model_runner import ModelRunner
    from nanovllm.engine.sequence import Sequence
    toks = [tokens_of(CFG_FLAT, n, 70 + n) for n in (30, 11, 21)]
    logits = {}
    for eager in (True, False):
        cfg = Config(flat_case.path, max_num_batched_tokens=64, max_num_seqs=4, max_model_len=128, num_kvcache_blocks=6, num_state_slots=4,
                     chunked_prefill=True, enforce_eager=eager, async_scheduling=False, dtype="float32")
        runner = ModelRunner(cfg, 0, [])
        try:
            seqs = []
            for i, t in enumerate(toks):
                s = Sequence(list(t[:-6]))
                s.block_table, s.state_slot, s.num_new_tokens = [i], i, len(t) - 6
                seqs.append(s)
            runner.forward_logits(seqs)
            rows = []
            for step in range(6):
                for s, t in zip(seqs, toks):
                    s.num_cached_tokens += s.num_new_tokens
                    s.append_token(t[len(t) - 6 + step])
                    s.num_new_tokens = 1
                out, _, _ = runner.forward_logits(seqs)
                rows.append(out.float().cpu().numpy())
            logits[eager] = np.stack(rows)
            assert eager or runner.graphs
        finally:
            runner.exit()
    assert np.abs(logits[True] - logits[False]).max() < 1e-4 * np.abs(logits[True]).max()
    for i, t in enumerate(toks):
        want = flat_case.ref(t)
        for step in range(6):
            assert rel_err(logits[False][step, i:i + 1], want[len(t) - 6 + step:len(t) - 5 + step]) < TOL["float32"]


def test_the_replay_program_steps_through_a_schedule(tmp_path, mix_case_calm):
    """bin/trace_run as a user starts it: steps on standard input, `done <n>` after each, logits of the wanted places in <out>/<n>.f32;
    a request that is left out of a step and goes on later, one that ends and whose pages and slot the next one takes over."""
    import subprocess
    import sys
    from conftest import ROOT
    a, b = tokens_of(CFG_MIX, 40, 91), tokens_of(CFG_MIX, 12, 92)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:25], "want": [0, 24]}], "end": []},
             {"step": 1, "entries": [{"id": "b", "tokens": b[:10], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": a[25:39], "want": [13]}, {"id": "b", "tokens": b[10:], "want": [1]}], "end": ["b"]},
             {"step": 3, "entries": [{"id": "a", "tokens": a[39:], "want": [0]}], "end": ["a"]}]
    for dtype in ("bfloat16", "float32"):
        out = tmp_path / dtype
        done = subprocess.run([sys.executable, str(ROOT / "bin" / "trace_run"), "--model", mix_case_calm.path, "--dtype", dtype, "--out", str(out), "--max-tokens", "128"],
                              input="".join(json.dumps(st) + "\n" for st in steps), capture_output=True, text=True, timeout=600)
        assert done.returncode == 0, done.stderr[-2000:]
        assert [ln for ln in done.stdout.splitlines() if ln.startswith("done")] == [f"done {n}" for n in range(4)]
        assert not (out / "1.f32").exists()
        ra, rb = mix_case_calm.ref(a), mix_case_calm.ref(b)
        want = {0: ra[[0, 24]], 2: np.concatenate([ra[38:39], rb[11:12]]), 3: ra[39:40]}
        for n, w in want.items():
            got = np.fromfile(out / f"{n}.f32", dtype="<f4").reshape(-1, CFG_MIX["vocab"])
            assert got.shape == w.shape and rel_err(got, w) < TOL[dtype], (dtype, n)
