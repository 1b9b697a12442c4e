"""Sokipel through the engine against the plain float64 restatement in tests/sokipel_reference.py.

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

import sokipel_reference as R

pytestmark = pytest.mark.gpu

BANDS = {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64}          # with base 500 over 12 dims: pairs in all three bands
MOE_A = {"kind": "moe", "expert": {"ff": 24, "limit": 0.7}, "router": {"experts": 6, "top": 2}}
MOE_B = {"kind": "moe", "expert": {"ff": 36, "limit": 2.5}, "router": {"experts": 7, "top": 3}}
MOE_C = {"kind": "moe", "expert": {"ff": 16, "limit": 1.5}, "router": {"experts": 5, "top": 1}}
# head sizes that no tile divides (the vector-ALU attention in both types), part of the head rotated, a chunk that is no multiple of anything
ATT_A = {"type": "attention", "mlp": MOE_A,
         "mixer": {"heads": 6, "kv_heads": 2, "dim": 20, "vdim": 12, "scale": 0.3, "rot": {"base": 500.0, "dims": 12, "scaling": BANDS}, "mask": {"size": 50}}}
# head sizes of 32 / 16 (the matrix-core attention in bf16), as many key heads as query heads, the whole head rotated
ATT_B = {"type": "attention", "mlp": None,
         "mixer": {"heads": 4, "kv_heads": 4, "dim": 32, "vdim": 16, "scale": 0.25, "rot": {"base": 10000.0, "dims": 32, "scaling": BANDS}, "mask": {"size": 37}}}
DEL_A = {"type": "delta", "mlp": MOE_B, "mixer": {"heads": 3, "kv_heads": 3, "dim": 20, "vdim": 28, "conv": 4}}
DEL_B = {"type": "delta", "mlp": None, "mixer": {"heads": 4, "kv_heads": 2, "dim": 32, "vdim": 16, "conv": 2}}
DEL_C = {"type": "delta", "mlp": MOE_C, "mixer": {"heads": 2, "kv_heads": 1, "dim": 6, "vdim": 5, "conv": 1}}
PAR_A = {"type": "parallel", "mlp": MOE_C,
         "mixer": {"left": {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 32, "scale": 0.3, "rot": {"base": 700.0, "dims": 8, "scaling": {"factor": 3.0}}},
                   "left_scale": 0.4, "right": {"heads": 2, "kv_heads": 1, "dim": 16, "vdim": 24, "conv": 3}, "right_scale": 1.3}}
PAR_B = {"type": "parallel", "mlp": None,
         "mixer": {"left": {"heads": 3, "kv_heads": 1, "dim": 12, "vdim": 20, "scale": 0.4, "rot": {"base": 90.0, "dims": 12}},
                   "left_scale": 1.1, "right": {"heads": 2, "kv_heads": 2, "dim": 10, "vdim": 10, "conv": 5}, "right_scale": 0.5}}


def config(layers, width=96, vocab=131, taps=3, scale=4.0, mult=0.6, cap=20.0, eps=1e-5):
    cfg = {"architecture": "Sokipel", "vocab": vocab, "width": width, "norm": {"eps": eps}, "embedding": {"scale": scale}, "residual_mult": mult,
           "logit_softcap": cap, "layers": copy.deepcopy(layers)}
    if taps:
        cfg["canon"] = {"taps": taps}
    return cfg


CFG_MIX = config([DEL_A, PAR_A, ATT_A, PAR_B, DEL_B])
CFG_FLAT = config([ATT_B, DEL_B, PAR_A, DEL_C], width=128, vocab=200, taps=5, scale=2.0, mult=0.5, cap=35.0, eps=1e-6)


def random_weights(cfg: dict, seed: int, calm: bool = False) -> dict:
    """bf16 weights in checkpoint naming; decays spread so that some heads forget fast and some hardly at all.  `calm`: every token
    carries one large constant coordinate on which alone the routers look, with weights that lie far apart, so that the rounding of
    bf16 serving cannot flip a choice (the lively router, whose choice follows the token, is for fp32 serving)."""
    g = torch.Generator().manual_seed(seed)
    D, V = cfg["width"], cfg["vocab"]
    W = {}

    def mat(name, out, inp, scale=None):
        W[name] = torch.randn(out, inp, generator=g) * (scale if scale is not None else 1.0 / math.sqrt(inp))

    def vec(name, n, scale=1.0, shift=0.0):
        W[name] = shift + scale * torch.randn(n, generator=g)

    def one(name, scale=0.2, shift=1.0):
        W[name] = shift + scale * torch.randn((), generator=g)

    def attention(p, m, beside):
        h, d = m["heads"], m["dim"]
        kv, dv = m.get("kv_heads", h), m.get("vdim", d)
        for leaf, n in (("q", h * d), ("k", kv * d), ("v", kv * dv)):
            mat(p + leaf, n, D, 0.5 / math.sqrt(D))
            if beside:
                vec(p + leaf + ".b", n, 0.3)
        vec(p + "q.norm", d if beside else h * d, 0.2, 1.0)
        vec(p + "k.norm", d if beside else kv * d, 0.2, 1.0)
        vec(p + "sink", h, 1.0, 1.0)
        if beside:
            mat(p + "g", h, D, 0.3 / math.sqrt(D))
        mat(p + "o", D, h * dv)

    def delta(p, m):
        h, d = m["heads"], m["dim"]
        kv, dv, taps = m.get("kv_heads", h), m.get("vdim", d), m["conv"]
        for leaf, n in (("q", kv * d), ("k", kv * d), ("v", h * dv)):
            mat(p + leaf, n, D, 0.5 / math.sqrt(D))
            W[p + leaf + ".conv"] = torch.randn(n, taps, generator=g) * 0.5
        mat(p + "b", h, D, 0.3 / math.sqrt(D))
        mat(p + "a", h, D, 0.3 / math.sqrt(D))
        W[p + "A_log"] = torch.linspace(-4.0, 0.5, h)[torch.randperm(h, generator=g)]
        vec(p + "dt_bias", h, 0.5, -1.0)
        vec(p + "norm", dv, 0.2, 1.0)
        mat(p + "g", h * dv, D, 0.3 / math.sqrt(D))
        mat(p + "o", D, h * dv)

    mat("embed", V, D, 1.0)
    if calm:
        W["embed"][:, 0] = 24.0 / cfg["embedding"]["scale"]            # (large beside what the layers add to it on the way)
    mat("head", V, D)
    one("final.norm")
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        one(p + "norm1")
        if cfg.get("canon"):
            W[p + "canon1"] = torch.randn(D, cfg["canon"]["taps"], generator=g) * 0.3
        if L["type"] == "attention":
            attention(p + "mix.", m, False)
        elif L["type"] == "delta":
            delta(p + "mix.", m)
        else:
            attention(p + "mix.left.", m["left"], True)
            delta(p + "mix.right.", m["right"])
        mlp = L.get("mlp")
        if not mlp:
            continue
        one(p + "norm2")
        E, ff = mlp["router"]["experts"], mlp["expert"]["ff"]
        for e in range(E):
            mat(f"{p}mlp.e{e}.gate", ff, D, 1.5 / math.sqrt(D))
            mat(f"{p}mlp.e{e}.up", ff, D, 1.5 / math.sqrt(D))
            mat(f"{p}mlp.e{e}.down", D, ff)
        if calm:
            mat(p + "mlp.router", E, D, 0.02 / math.sqrt(D))
            W[p + "mlp.router"][:, 0] = torch.linspace(-0.15, 0.15, E)[torch.randperm(E, generator=g)]
        else:
            mat(p + "mlp.router", E, D, 0.5 / math.sqrt(D))
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
    return Case(tmp_path_factory.mktemp("sokipel_mix"), CFG_MIX, seed=1)


@pytest.fixture(scope="module")
def mix_case_calm(tmp_path_factory):
    return Case(tmp_path_factory.mktemp("sokipel_mix_calm"), CFG_MIX, seed=1, calm=True)


@pytest.fixture(scope="module")
def flat_case(tmp_path_factory):
    return Case(tmp_path_factory.mktemp("sokipel_flat"), CFG_FLAT, seed=2, calm=True)


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
@pytest.mark.parametrize("layer", [ATT_A, ATT_B, DEL_A, DEL_B, DEL_C, PAR_A, PAR_B],
                         ids=["attention(ragged, part rotated, banded frequencies)+moe", "attention(matrix cores in bf16)", "delta(ragged)+moe", "delta(exact, grouped keys)",
                              "delta(one tap, one small key head)+moe", "parallel(interpolated positions)+moe", "parallel(ragged, five taps)"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_one_layer_stream_matches(tmp_path, layer, dtype):
    """One layer of each kind: the residual stream after it and the logits; 70 tokens cross the chunk's edge."""
    cfg = config([layer], width=72, vocab=50, taps=4, mult=0.8)
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


def test_every_layer_of_a_stack(mix_case):
    toks = tokens_of(CFG_MIX, 60, 7)
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


def test_a_stack_without_the_stream_convolution(tmp_path):
    """No `canon` in the config: every sublayer reads the stream as it is (its copy in the activation type comes from the closing kernels)."""
    cfg = config([DEL_B, ATT_A, PAR_B], taps=0)
    for dtype in ("float32", "bfloat16"):
        case = Case(tmp_path / dtype, cfg, seed=8, calm=dtype == "bfloat16")
        toks = tokens_of(cfg, 66, 9)
        rp = case.replay(dtype)
        try:
            run_schedule(rp, case, {"a": toks}, [[("a", 40)], [("a", 25)], [("a", 1)]], dtype)
        finally:
            rp.close()


def test_gated_delta_scan_against_the_recurrence():
    """The prep and the scan against the recurrence written out: key sizes that are and are not multiples of 16 and of 4, value sizes
    of their own, grouped key heads, one to five taps; one sequence continued from a state and carried convolution inputs, one fresh,
    slots out of order; then the shape of a captured decode step with a padded row."""
    from nanovllm import ops
    g = torch.Generator().manual_seed(0)
    for H, G, dk, dv, taps, lens in [(3, 3, 20, 28, 4, [9, 5]), (4, 2, 32, 16, 2, [9, 5]), (2, 1, 6, 5, 1, [9, 5]), (2, 2, 48, 48, 3, [70, 3]), (1, 1, 37, 9, 5, [2, 40]),
                                     (6, 2, 16, 130, 3, [33, 1]), (1, 1, 128, 64, 4, [12, 12])]:
        past = [4, 0]
        T, C = sum(lens), 2 * G * dk + H * dv
        proj = torch.randn(T, C + 2 * H, generator=g)
        conv_w = torch.randn(C, taps, generator=g) * 0.5
        dt_bias, a_log = torch.randn(H, generator=g), torch.randn(H, generator=g) * 0.7 - 1.0
        state = torch.randn(5, H, dk, dv, generator=g)
        carried = torch.randn(5, max(taps - 1, 1), C, generator=g)
        slots = [3, 1]
        want, new_state, new_carried = torch.zeros(T, H * dv, dtype=torch.float64), state.double().clone(), carried.double().clone()
        t0 = 0
        for b, n in enumerate(lens):
            rows = proj[t0:t0 + n, :C].double()
            before = carried[slots[b], :taps - 1].double() if (past[b] and taps > 1) else torch.zeros(taps - 1, C, dtype=torch.float64)
            both = torch.cat([before, rows])
            act = torch.stack([R.silu((conv_w.double().T * both[t:t + taps]).sum(0)) for t in range(n)])
            if taps > 1:
                new_carried[slots[b], :taps - 1] = both[-(taps - 1):]
            q, k, v = act[:, :G * dk].view(n, G, dk), act[:, G * dk:2 * G * dk].view(n, G, dk), act[:, 2 * G * dk:].view(n, H, dv)
            q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) / math.sqrt(dk)
            k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
            beta = torch.sigmoid(proj[t0:t0 + n, C:C + H].double())
            dec = torch.exp(-torch.exp(a_log.double()) * torch.nn.functional.softplus(proj[t0:t0 + n, C + H:].double() + dt_bias.double()))
            for h in range(H):
                S = state[slots[b], h].double() if past[b] else torch.zeros(dk, dv, dtype=torch.float64)
                kh = h // (H // G)
                for t in range(n):
                    S = dec[t, h] * S
                    S = S + torch.outer(k[t, kh], beta[t, h] * (v[t, h] - S.T @ k[t, kh]))
                    want[t0 + t, h * dv:(h + 1) * dv] = S.T @ q[t, kh]
                new_state[slots[b], h] = S
            t0 += n
        st, cs, pj = state.clone().cuda(), carried.clone().cuda(), proj.cuda()
        cu = torch.tensor([0, lens[0], T], dtype=torch.int32).cuda()
        ctx = torch.tensor([lens[0] + past[0], lens[1] + past[1]], dtype=torch.int32).cuda()
        got = ops.gated_delta_rule(pj[:, :C], pj[:, C:C + H], pj[:, C + H:], conv_w.cuda(), dt_bias.cuda(), a_log.cuda(), cs, st,
                                   torch.tensor(slots, dtype=torch.int32).cuda(), cu, ctx, H, G, dk, dv)
        assert (got.cpu().double() - want).abs().max() < 1e-4 * max(1.0, float(want.abs().max())), (H, G, dk, dv, taps)
        assert (st.cpu().double() - new_state).abs().max() < 1e-4 * max(1.0, float(new_state.abs().max()))
        if taps > 1:
            assert torch.equal(cs.cpu().double()[:, :taps - 1], new_carried[:, :taps - 1])
        # one token per sequence, no offsets; the middle row is padding (slot -1) and touches no state
        st2, cs2 = st.clone(), cs.clone()
        one = ops.gated_delta_rule(pj[:3, :C], pj[:3, C:C + H], pj[:3, C + H:], conv_w.cuda(), dt_bias.cuda(), a_log.cuda(), cs2, st2,
                                   torch.tensor([3, -1, 0], dtype=torch.int32).cuda(), None, torch.tensor([50, 0, 1], dtype=torch.int32).cuda(), H, G, dk, dv)
        assert torch.isfinite(one.cpu()[[0, 2]]).all() and torch.equal(st2.cpu()[[1, 2, 4]], st.cpu()[[1, 2, 4]]) and not torch.equal(st2.cpu()[3], st.cpu()[3])


def test_stream_convolution_takes_earlier_rows_from_the_step_or_the_slot():
    from nanovllm import ops
    g = torch.Generator().manual_seed(4)
    for dim, taps in [(37, 4), (96, 2), (520, 5), (8, 1)]:
        x, w = torch.randn(8, dim, generator=g), torch.randn(dim, taps, generator=g)
        state = torch.randn(4, max(taps - 1, 1), dim, generator=g)
        # sequence 0: 5 tokens continued (slot 2 holds its last rows); sequence 1: 3 tokens, fresh, in slot 0
        st = state.clone().cuda()
        cu, ctx = torch.tensor([0, 5, 8], dtype=torch.int32).cuda(), torch.tensor([9, 3], dtype=torch.int32).cuda()
        for cast, tol in ((torch.float32, 1e-5), (torch.bfloat16, 0.06)):
            st = state.clone().cuda()
            out = ops.stream_conv(x.cuda(), w.to(cast).cuda(), st, torch.tensor([2, 0], dtype=torch.int32).cuda(), cu, ctx).cpu()
            wd = w.to(cast).double()
            a = torch.cat([state[2, :taps - 1].double(), x[:5].double()])
            b = torch.cat([torch.zeros(taps - 1, dim, dtype=torch.float64), x[5:].double()])
            want = torch.cat([torch.stack([s[t + taps - 1] + (wd.T * s[t:t + taps]).sum(0) for t in range(n)]) for s, n in ((a, 5), (b, 3))])
            assert out.dtype == cast and (out.double() - want).abs().max() < tol * max(1.0, float(want.abs().max())), (dim, taps)
            if taps > 1:
                assert torch.equal(st.cpu()[2, :taps - 1].double(), a[-(taps - 1):]) and torch.equal(st.cpu()[0, :taps - 1].double(), b[-(taps - 1):])
                assert torch.equal(st.cpu()[1], state[1])


def test_sublayer_norm_kernel_against_its_formula():
    from nanovllm import ops
    g = torch.Generator().manual_seed(3)
    unit = lambda v: v / torch.sqrt((v * v).mean(-1, keepdim=True) + 1e-5)
    for dim in (50, 96, 1000):
        x, a, b, c = (torch.randn(9, dim, generator=g) for _ in range(4))
        w1, wn = torch.tensor([1.7]), torch.randn(dim, generator=g)
        xg = x.cuda()
        h = ops.residual_subnorm(xg, w1.cuda(), 1e-5, 0.6, a=a.cuda(), a_scale=0.4, b=b.cuda(), b_scale=1.3)
        want = x + 0.6 * 1.7 * unit(0.4 * a + 1.3 * b)
        assert (xg.cpu() - want).abs().max() < 1e-5 and (h.cpu() - want).abs().max() < 1e-5
        xg = x.cuda()
        assert ops.residual_subnorm(xg, wn.cuda(), 1e-5, 1.0, c32=c.cuda(), want_h=False) is None          # a weight per column, the fp32 term alone
        assert (xg.cpu() - (x + wn * unit(c))).abs().max() < 1e-5
        xg = x.cuda()
        hb = ops.residual_subnorm(xg, w1.bfloat16().cuda(), 1e-5, 0.6, a=a.bfloat16().cuda(), c32=c.cuda())
        want = x + 0.6 * w1.bfloat16().float() * unit(a.bfloat16().float() + c)
        assert hb.dtype == torch.bfloat16 and (xg.cpu() - want).abs().max() < 1e-5 and (hb.float().cpu() - want).abs().max() < 0.05


def test_sigmoid_router_and_the_capped_unit_with_the_weight_on_the_input():
    from nanovllm import ops
    g = torch.Generator().manual_seed(1)
    for E, top in [(6, 2), (7, 3), (5, 1), (64, 6), (130, 8), (3, 3), (1, 1)]:
        x, w = torch.randn(33, 70, generator=g), torch.randn(E, 70, generator=g) * 0.3
        for cast in (torch.float32, torch.bfloat16):
            xa, wa = x.to(cast), w.to(cast)
            s = torch.sigmoid(xa.double() @ wa.double().T)
            idx = s.topk(top, -1).indices
            ids, wts = ops.moe_route_linear(xa.cuda(), wa.cuda(), None, top, sigmoid_scores=True)
            assert torch.equal(ids.cpu().long(), idx), (E, top)
            assert (wts.cpu().double() - s.gather(1, idx)).abs().max() < 1e-5
    T, E, top, ff = 40, 5, 2, 52
    ids = torch.randint(0, E, (T, top), generator=g).int()
    wts = torch.rand(T, top, generator=g)
    gu = torch.randn(T * top, 2 * ff, generator=g) * 2
    plan = ops.moe_align(ids.cuda(), E)
    pos = plan["pos_of_pair"].cpu().long()
    for limit, alpha in ((0.7, 1.702), (2.5, 1.0)):
        y = ops.glu_clamp_pairs(gu.cuda(), plan, wts.cuda(), limit, alpha).cpu()
        scaled = gu[pos] * wts.view(-1, 1)
        a, b = scaled[:, :ff].clamp(max=limit), scaled[:, ff:].clamp(-limit, limit)
        assert (y[pos] - a * torch.sigmoid(alpha * a) * (b + 1)).abs().max() < 1e-5
    rows = torch.randn(T * top, 30, generator=g)
    assert (ops.moe_combine(rows.cuda(), plan, None, top=top).cpu() - rows[pos.view(T, top)].sum(1)).abs().max() < 1e-5


def test_attention_with_sinks_and_chunks_against_dense_softmax():
    """The paged attention with a sink per head and chunks, prompts cut into steps and one-query steps (where, in bf16, the heads of a
    group share a workgroup and a sequence's key tiles go to several): sizes for the matrix-core and for the vector-ALU kernel."""
    from nanovllm import ops
    g = torch.Generator().manual_seed(6)
    page = 256
    for H, G, d, dv, chunk in [(4, 2, 32, 16, 100), (6, 2, 20, 12, 37), (2, 2, 64, 64, 0), (8, 1, 16, 32, 300)]:
        for cast, tol in ((torch.float32, 1e-4), (torch.bfloat16, 2e-2)):
            lens = [530, 70]
            q = [torch.randn(n, H, d, generator=g).to(cast) for n in lens]
            k = [torch.randn(n, G, d, generator=g).to(cast) for n in lens]
            v = [torch.randn(n, G, dv, generator=g).to(cast) for n in lens]
            sinks = torch.randn(H, generator=g) * 2 + 2
            want = [R.sink_softmax_attention(a.double(), b.double(), c.double(), 0.3, sinks.double(), chunk) for a, b, c in zip(q, k, v)]
            kc, vc = torch.zeros(5, page, G, d, dtype=cast), torch.zeros(5, G, dv, page, dtype=cast)
            pages = [[4, 0, 2], [1, 0, 0]]
            for b, n in enumerate(lens):
                for t in range(n):
                    kc[pages[b][t // page], t % page] = k[b][t]
                    vc[pages[b][t // page], :, :, t % page] = v[b][t]
            kc, vc, tables = kc.cuda(), vc.cuda(), torch.tensor(pages, dtype=torch.int32).cuda()
            # a step that brings the last 40 queries of the first sequence and all of the second; then one query of each
            for take in ((40, 70), (1, 1)):
                ends = [lens[0] - (5 if take[0] == 1 else 0), lens[1] - (9 if take[1] == 1 else 0)]
                qs = torch.cat([q[b][ends[b] - take[b]:ends[b]] for b in range(2)]).reshape(-1, H * d).cuda()
                cu = torch.tensor([0, take[0], take[0] + take[1]], dtype=torch.int32).cuda()
                out = ops.attn_paged_any(qs, kc, vc, cu if take[0] > 1 else None, torch.tensor(ends, dtype=torch.int32).cuda(), tables, 0.3, H, G, d, dv,
                                         chunk=chunk, sinks=sinks.cuda()).cpu().double()
                ref = torch.cat([want[b][ends[b] - take[b]:ends[b]] for b in range(2)]).reshape(-1, H * dv)
                assert (out - ref).abs().max() < tol * max(1.0, float(ref.abs().max())), (H, G, d, dv, chunk, cast, take)


# ----------------------------------------------------------------------------------------------------- schedules
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prefill_then_token_by_token(mix_case, mix_case_calm, dtype):
    mix_case = case_for(dtype, mix_case, mix_case_calm)
    toks = tokens_of(CFG_MIX, 120, 11)
    rp = mix_case.replay(dtype)
    try:
        run_schedule(rp, mix_case, {"a": toks}, [[("a", 45)]] + [[("a", 1)]] * 75, dtype)          # decoding across two chunk edges (50, 100)
        # the first tokens of a sequence, one by one from the very start (no earlier rows to convolve, empty memories, one key)
        run_schedule(rp, mix_case, {"b": toks[:20]}, [[("b", 1)]] * 20, dtype)
    finally:
        rp.close()


def test_portions_of_every_size_give_the_same_logits(mix_case):
    toks = tokens_of(CFG_MIX, 120, 13)
    rp = mix_case.replay("float32")
    try:
        for sizes in ([120], [2] * 60, [3, 2, 17, 2, 33, 16, 2, 45], [64, 56], [1, 119], [49, 1, 1, 49, 2, 18]):
            assert sum(sizes) == 120
            run_schedule(rp, mix_case, {"a": toks}, [[("a", s)] for s in sizes], "float32")
    finally:
        rp.close()


def test_cutting_does_not_change_a_bit_of_the_recurrent_path(tmp_path):
    """Delta-rule layers only (no attention, whose key tiles see the cut): one piece, portions and single tokens give identical
    logits, the carried convolution inputs included."""
    cfg = config([DEL_A, DEL_B, DEL_C], width=64, vocab=64, taps=4)
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
    the first two runs on pages and slots (memories, carried rows) that others have left behind."""
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
def test_page_borders_and_chunk_edges_in_prompts_and_in_decoding(flat_case, dtype):
    """Portions that end one token before, at and after a page border, then decoding across the next one; portions that end one
    token before, at and after an edge of the 37-token chunks."""
    toks = tokens_of(CFG_FLAT, 530, 41)
    rp = flat_case.replay(dtype, max_tokens=1100)
    try:
        run_schedule(rp, flat_case, {"a": toks}, [[("a", 255)], [("a", 1)], [("a", 1)], [("a", 2)], [("a", 251)], [("a", 3)]] + [[("a", 1)]] * 17, dtype)
        for first in (36, 37, 38, 73, 74, 75, 256, 257):
            run_schedule(rp, flat_case, {"b": toks[:first + 8]}, [[("b", first)], [("b", 7)], [("b", 1)]], dtype)
    finally:
        rp.close()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_one_token_steps_of_sequences_of_unequal_length(flat_case, dtype):
    """Steps in which every sequence brings one token: contexts of one to five key tiles side by side; then fewer sequences as the
    short requests end."""
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
def sharp_attention_case(tmp, beside: bool, chunk: int):
    """One layer without the stream convolution whose keys equal its queries (same projection, same norm, no rotation) under a large
    scale: a query puts nearly all its weight on itself and on the earlier occurrence of its own token.  `beside`: the attention of a
    parallel mixer (every earlier token visible; the delta rule beside it counts little); else the chunked one."""
    att = {"heads": 2, "kv_heads": 2, "dim": 32, "vdim": 32, "scale": 0.5}
    if beside:
        layer = {"type": "parallel", "mlp": None, "mixer": {"left": att, "left_scale": 1.0, "right": {"heads": 1, "kv_heads": 1, "dim": 16, "vdim": 16, "conv": 2}, "right_scale": 0.05}}
    else:
        layer = {"type": "attention", "mlp": None, "mixer": dict(att, mask={"size": chunk})}
    cfg = config([layer], width=64, vocab=900, taps=0, scale=3.0, mult=1.0)
    w = random_weights(cfg, 9)
    p = "l0.mix.left." if beside else "l0.mix."
    w[p + "k"] = w[p + "q"].clone()
    w[p + "k.norm"] = w[p + "q.norm"].clone()
    if beside:
        w[p + "k.b"] = w[p + "q.b"].clone()
    w[p + "sink"] = torch.tensor([10.0, 19.0]).to(w[p + "sink"].dtype)      # light beside a matching key in one head, heavier than it in the other: leaving it out would show
    w[p + "v"] = w[p + "v"] * 4
    return Case(tmp, cfg, weights=w), cfg


@pytest.mark.parametrize("beside", [False, True], ids=["chunked", "beside a delta rule"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_far_key_decides_wherever_it_lies(tmp_path, dtype, beside):
    """The last token repeats an earlier one, which then gets much of the weight among 600 keys: at the start, around both page
    borders, right before the query - and, with chunks of 200, at the chunk's first position but not one before it.  Whole prompt
    in one step, and the last token decoded alone.  The sink shows as well."""
    case, cfg = sharp_attention_case(tmp_path, beside, 200)
    n = 600
    base = list(range(1, n + 1))
    plain = case.ref(base[:n - 1] + [899])[-1:]
    W = dict(case.W)
    sink = "l0.mix.left.sink" if beside else "l0.mix.sink"
    W[sink] = torch.full_like(W[sink], -30.0)
    assert rel_err(R.forward(W, cfg, base[:n - 1] + [899]).numpy()[-1:], plain) > 0.05          # without the sink the logits are others
    rp = case.replay(dtype, max_tokens=1300)
    try:
        for far in (0, 3, 255, 256, 257, 399, 400, 401, 511, 512, n - 2):
            toks = base[:n - 1] + [base[far]]
            ref = case.ref(toks)[-1:]
            seen = beside or far >= 400
            other = case.ref(base[:n - 1] + [899])[-1:] if seen else case.ref(base[:far] + [898] + base[far + 1:n - 1] + [base[far]])[-1:]
            if seen:
                assert rel_err(other, ref) > 0.2, far          # the key matters: without it the logits are others
            else:
                assert rel_err(other, ref) < 1e-9, far         # a key before the chunk: whatever stands there, the logits are the same
            whole = rp.step([{"id": 0, "tokens": toks, "want": [n - 1]}], [0])
            rp.step([{"id": 1, "tokens": toks[:n - 1], "want": []}])
            decoded = rp.step([{"id": 1, "tokens": toks[n - 1:], "want": [0]}], [1])
            tol = TOL[dtype] if dtype == "float32" else 0.15      # (sharp weights magnify the rounding of bf16 scores)
            assert rel_err(whole, ref) < tol and rel_err(decoded, ref) < tol, far
    finally:
        rp.close()


def test_the_memory_carries_a_token_from_far_back(tmp_path):
    """Decays near one keep the delta rule's memory for hundreds of tokens: the first token still shapes the last logits, and a state
    that were lost or reset between portions would show."""
    layer = {"type": "delta", "mlp": None, "mixer": {"heads": 2, "kv_heads": 1, "dim": 16, "vdim": 24, "conv": 3}}
    cfg = config([layer], width=48, vocab=90, taps=2, mult=1.0)
    w = random_weights(cfg, 4, calm=True)                              # (every token carries the constant first coordinate)
    w["l0.mix.A_log"] = torch.full_like(w["l0.mix.A_log"], -7.0)
    w["l0.canon1"][0] = 0
    w["l0.mix.b"] = w["l0.mix.b"] * 0.1
    w["l0.mix.b"][:, 0] = -0.2                                          # weak writes: a write also wears off what lies along its key
    case = Case(tmp_path, cfg, weights=w)
    toks = tokens_of(cfg, 400, 8)
    changed = [(toks[0] + 1) % 90] + toks[1:]
    assert rel_err(case.ref(changed)[-1:], case.ref(toks)[-1:]) > 5 * TOL["float32"]      # 400 tokens later it still shows
    rp = case.replay("float32", max_tokens=1024)
    try:
        run_schedule(rp, case, {"a": toks}, [[("a", 100)], [("a", 156)], [("a", 1)], [("a", 140)], [("a", 2)], [("a", 1)]], "float32")
        run_schedule(rp, case, {"b": toks, "c": toks[:9]}, [[("b", 290), ("c", 8)], [("b", 109), ("c", 1)], [("b", 1)]], "float32")
    finally:
        rp.close()


def test_the_weight_on_the_input_and_the_convolutions_show(tmp_path):
    """With the routing weight moved to the expert's result, or without the stream's convolution, the reference itself changes clearly,
    so the agreement of the other tests is not one that these faults could share."""
    cfg = config([DEL_A], width=48, vocab=90)
    case = Case(tmp_path, cfg, seed=4)
    toks = tokens_of(cfg, 30, 1)
    full = case.ref(toks)
    W = dict(case.W)
    W["l0.canon1"] = torch.zeros_like(W["l0.canon1"])
    assert rel_err(R.forward(W, cfg, toks).numpy(), full) > 0.05
    keep = R.experts

    def weight_after(Wt, p, mlp, x):
        cap = mlp["expert"]["limit"]
        score = torch.sigmoid(x @ Wt[p + "router"].T)
        y = torch.zeros_like(x)
        for t in range(x.shape[0]):
            for e in torch.topk(score[t], mlp["router"]["top"]).indices.tolist():
                a = torch.clamp(Wt[f"{p}e{e}.gate"] @ x[t], max=cap)
                b = torch.clamp(Wt[f"{p}e{e}.up"] @ x[t], min=-cap, max=cap)
                y[t] += score[t, e] * (Wt[f"{p}e{e}.down"] @ (a * torch.sigmoid(1.702 * a) * (b + 1.0)))
        return y
    R.experts = weight_after
    try:
        assert rel_err(R.forward(case.W, cfg, toks).numpy(), full) > 0.02
    finally:
        R.experts = keep


# ----------------------------------------------------------------------------------------------------- other sizes
def test_sizes_no_kernel_tile_divides(tmp_path):
    """A width that is no multiple of 8; one expert of which one is taken; twenty query heads over one key head (more than a one-token
    step shares a workgroup among); one head; a chunk of one token and one longer than the sequence; a two-wide rotated part; key
    sizes of 72 and 130 in the delta rule with a value size of 3; six taps."""
    one = {"kind": "moe", "expert": {"ff": 10, "limit": 0.5}, "router": {"experts": 1, "top": 1}}
    layers = [{"type": "attention", "mlp": one, "mixer": {"heads": 20, "kv_heads": 1, "dim": 4, "vdim": 4, "scale": 0.5, "rot": {"base": 50.0, "dims": 2}, "mask": {"size": 1}}},
              {"type": "delta", "mlp": {"kind": "moe", "expert": {"ff": 12, "limit": 3.0}, "router": {"experts": 4, "top": 4}}, "mixer": {"heads": 1, "kv_heads": 1, "dim": 130, "vdim": 3, "conv": 6}},
              {"type": "attention", "mlp": None, "mixer": {"heads": 1, "kv_heads": 1, "dim": 50, "vdim": 70, "scale": 0.1, "mask": {"size": 5000}}},
              {"type": "parallel", "mlp": None,
               "mixer": {"left": {"heads": 5, "kv_heads": 5, "dim": 10, "vdim": 6, "scale": 1.0, "rot": {"base": 3.0, "dims": 10, "scaling": {"factor": 1.0}}}, "left_scale": 2.0,
                         "right": {"heads": 3, "kv_heads": 1, "dim": 72, "vdim": 10, "conv": 2}, "right_scale": 1.0}}]
    cfg = config(layers, width=50, vocab=37, taps=6, scale=1.0, mult=1.0, cap=0.0)
    del cfg["logit_softcap"]
    case = Case(tmp_path, cfg, weights=random_weights(cfg, 6, calm=True))
    toks = tokens_of(cfg, 80, 3)
    for dtype in ("float32", "bfloat16"):
        rp = case.replay(dtype)
        try:
            run_schedule(rp, case, {"a": toks, "b": toks[:7]}, [[("a", 33), ("b", 5)], [("a", 1), ("b", 2)], [("a", 44)], [("a", 1)], [("a", 1)]], dtype,
                         tol=None if dtype == "float32" else 0.15)     # (50 columns wide: the rounding of bf16 adds up layer by layer)
        finally:
            rp.close()
    with pytest.raises(ValueError):
        from nanovllm.models.sokipel import SokipelForCausalLM
        from types import SimpleNamespace
        SokipelForCausalLM(SimpleNamespace(**config([dict(DEL_B, type="unknown")])))


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
    """One-token steps replayed from the captured graph (routing, expert tiles, states and carried rows inside it) against the
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


def test_the_sample_config_is_served_with_random_weights():
    """model_configs/sokipel-mixed-1k (layer sizes of a real model; no checkpoint, so the engine draws weights): prompts of unequal
    length are prefilled in chunks and decoded from captured graphs."""
    from conftest import ROOT
    from nanovllm import LLM, SamplingParams
    llm = LLM(str(ROOT / "nano-vllm-v1_amd" / "model_configs" / "sokipel-mixed-1k"), max_num_seqs=4, max_num_batched_tokens=256, max_model_len=1024,
              num_kvcache_blocks=12, chunked_prefill=True)
    try:
        prompts = [torch.randint(0, 32768, (n,), generator=torch.Generator().manual_seed(n)).tolist() for n in (600, 3, 130)]
        outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=8, ignore_eos=True), use_tqdm=False)
        again = llm.generate(prompts[1:2], SamplingParams(temperature=0.0, max_tokens=8, ignore_eos=True), use_tqdm=False)
    finally:
        llm.exit()
    assert all(len(o["token_ids"]) == 8 for o in outs) and again[0]["token_ids"] == outs[1]["token_ids"]
