"""The Malinex decoder on the GPU against the plain implementation (plain_malinex.py): each mechanism alone, then
the engine on small models of other sizes than any real one: whole prompts, the tail decoded token by token,
portions down to two tokens, mixed batches over pools so small that pages and state slots are used again (freed
pages hold NaN), a key that stands out far back, at a page's border and at the causal edge, a state that reaches
hundreds of tokens back, long decoding from graphs, and greedy generation through the runtime and its scheduler."""
import math

import pytest
import torch

import malinex_models as MM
import plain_malinex as PM
import trace_tools as TT
from part_harness import DEV, TOL as PART_TOL, Steps, build, dense, rel_err, runtime

pytestmark = pytest.mark.gpu
BOTH = pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
# largest |difference| of a logit as a fraction of the RMS of the plain logits
TOL = {"float32": 3e-5, "bfloat16": 6e-2}
NAMES = ["X1", "X2", "X3", "X4", "X5"]
LENGTHS = {"X1": (1, 7, 45, 83, 130), "X2": (3, 61, 33, 97), "X3": (9, 70, 121), "X4": (2, 17, 64, 150), "X5": (1, 64, 65, 140)}
MIXED = {"X1": (70, 131, 64, 150, 33, 97, 66, 81), "X2": (150, 165, 120, 190, 147), "X3": (129, 65, 90, 47, 72, 99),
         "X4": (70, 131, 64, 150, 33, 97), "X5": (150, 100, 64, 190, 129, 77)}
PAGE = {"X1": 16, "X2": 4, "X3": 8, "X4": 16, "X5": 12}
# In bfloat16 a router's close call may fall the other way than in the plain model (its input is the rounded
# stream); the token then takes another expert, and the recurrent state and the keys carry that to every later
# place: places from a request's first such call on (a margin below this in the plain model) are held to be finite
# only.  The 32-bit path is held at every place; the routed layer alone in test_routed_experts.
CLOSE_CALL = 0.1
BF16_TOL = {}
EPS = 1e-5


def _x(n, h, dtype, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(n, h, generator=g) * scale
    return x.to(torch.bfloat16).float() if dtype == "bfloat16" else x


def _tol(dtype, want, rounded):
    """Three times what rounding every stored activation to bfloat16 costs the plain form, and at least the parts'
    usual tolerance; in 32-bit the parts' usual one."""
    if dtype != "bfloat16":
        return PART_TOL[dtype]
    return max(PART_TOL[dtype], 3.0 * rel_err(rounded().to(torch.bfloat16), want))


def _mixer_weights(kind, m, W, seed):
    cfg = {"vocab": 4, "width": W, "max_positions": 4, "norm": {"eps": EPS}, "layers": [{"type": kind, "mixer": m, "mlp": None}]}
    return {k[len("l0.mix."):]: v.double() for k, v in PM.random_weights(cfg, seed).items() if k.startswith("l0.mix.")}


def _gla_params(m, W):
    return {"hidden_size": W, "num_heads": m["heads"], "head_dim": m["dim"], "value_dim": m["vdim"], "tau": m["tau"],
            "decay_rank": m["rank"], "norm_eps": EPS}


def _att_params(m, W):
    return {"hidden_size": W, "num_heads": m["heads"], "num_kv_heads": m.get("kv_heads", m["heads"]), "head_dim": m["dim"],
            "value_dim": m["vdim"], "scale": m["scale"], "norm_eps": EPS, "q_temp": m.get("q_temp")}


def _run_mixer(mixer, steps, x, cuts, rt, request="a"):
    """Feeds x [T, W] of one request through the mixer in the portions ``cuts``."""
    out, p = [], 0
    for n in cuts:
        ctx, packed = steps.begin([(request, n)])
        out.append(dense(mixer.forward(x[p:p + n].to(DEV).to(rt.dtype), ctx, steps.views[0]), rt).float().cpu())
        steps.end(packed)
        p += n
    assert p == x.shape[0]
    return torch.cat(out)


# ------------------------------------------------------------------------------------ kernels alone
@BOTH
def test_learned_position_rows(dtype):
    from infernum_amd.kernels import api as K
    rt = runtime(dtype)
    g = torch.Generator().manual_seed(1)
    table, pos_table = torch.randn(50, 72, generator=g), torch.randn(40, 72, generator=g)
    if dtype == "bfloat16":
        table, pos_table = table.to(torch.bfloat16).float(), pos_table.to(torch.bfloat16).float()
    toks = torch.randint(0, 50, (23,), generator=g)
    pos = torch.tensor([0, 1, 2, 39, 38, 5, 5, 0] + list(range(10, 25)))
    h = torch.empty((23, 72), dtype=torch.float32, device=DEV)
    K.embed(table.to(DEV).to(rt.dtype), toks.to(DEV).int(), h, 1.0)
    K.add_rows(h, pos_table.to(DEV).to(rt.dtype), pos.to(DEV).int())
    want = PM.embed(toks, table.double(), pos, pos_table.double())
    assert rel_err(h, want) <= 1e-6


@BOTH
@pytest.mark.parametrize("N,H,splits", [(1, 64, 0), (9, 100, 0), (70, 256, 3), (5, 48, 2), (300, 2048, 0), (3, 4100, 2), (4, 6, 0), (2, 16388, 0)])
@pytest.mark.parametrize("gated,nxt", [(True, True), (True, False), (False, True)])
def test_gated_branch_norm(dtype, N, H, splits, gated, nxt):
    """h += norm(delta * sigmoid(G + b)) and, with a next norm, its rows besides; the delta a tensor or partial sums."""
    from infernum_amd.kernels import api as K
    rt = runtime(dtype)
    g = torch.Generator().manual_seed(N + H)
    h = torch.randn(N, H, generator=g)
    parts = torch.randn(max(splits, 1), N, H, generator=g)
    delta = parts.sum(0) if splits else _x(N, H, dtype, 4)
    gate, bias = torch.randn(N, H, generator=g) * 2, torch.randn(H, generator=g)
    gate_parts = None
    if gated and splits:                              # the gate's logits as the parts of a split product too
        gate_parts = torch.randn(splits, N, H, generator=g)
        gate = gate_parts[0].clone()
        for k in range(1, splits):
            gate = gate + gate_parts[k]
    w, w2 = torch.rand(H, generator=g) + 0.5, torch.rand(H, generator=g) + 0.5
    d = delta.double() * (PM.sigmoid(gate.double() + bias.double()) if gated else 1.0)
    want_h = h.double() + PM.rms_norm(d, w.double(), EPS)
    want_x = PM.rms_norm(want_h, w2.double(), EPS)
    hd = h.clone().to(DEV)
    xd = torch.empty((N, H), dtype=rt.dtype, device=DEV) if nxt else None
    dd = K.SplitSum(parts.to(DEV)) if splits else delta.to(DEV).to(rt.dtype)
    gd = K.SplitSum(gate_parts.to(DEV)) if gate_parts is not None else (gate.to(DEV) if gated else None)
    K.gated_norm_add(hd, dd, gd, bias.to(DEV) if gated else None, w.to(DEV), EPS,
                     w2.to(DEV) if nxt else None, xd)
    assert rel_err(hd, want_h) <= 2e-5
    if nxt:
        assert rel_err(xd, want_x) <= PART_TOL[dtype]


@pytest.mark.parametrize("N,E,top", [(1, 6, 2), (40, 5, 5), (33, 70, 1), (200, 12, 4), (7, 128, 8), (5, 3, 1)])
def test_router_softmax_first(N, E, top):
    """A softmax over all experts, the choice by score + correction, the weights the chosen scores over their sum."""
    from infernum_amd.kernels import api as K
    g = torch.Generator().manual_seed(E + top)
    z, corr = torch.randn(N, E, generator=g) * 2, torch.randn(E, generator=g) * 0.1
    ids, wts = K.router_softmax_topk(z.to(DEV), corr.to(DEV), top)
    margins = []
    chosen, want = PM.router(z.double(), torch.eye(E, dtype=torch.float64), corr.double(), top, margins)
    sure = margins[0] > 1e-4 if margins else torch.ones(N, dtype=torch.bool)
    assert sure.sum() >= N * 0.8
    for n in range(N):
        if not sure[n]:
            continue
        got = dict(zip(ids[n].tolist(), wts[n].tolist()))
        ref = dict(zip(chosen[n].tolist(), want[n].tolist()))
        assert set(got) == set(ref) and len(got) == top
        assert all(abs(got[e] - ref[e]) <= 1e-6 for e in ref)
    # the correction moves the choice only: with a large one on an unlikely expert that expert is chosen and
    # weighs what its own small score gives it
    corr2 = torch.zeros(E)
    corr2[E - 1] = 5.0
    ids2, wts2 = K.router_softmax_topk(z.to(DEV), corr2.to(DEV), top)
    s = torch.softmax(z.double(), -1)
    for n in range(N):
        got = dict(zip(ids2[n].tolist(), wts2[n].tolist()))
        assert E - 1 in got
        assert abs(got[E - 1] - float(s[n, E - 1] / s[n, list(got)].sum())) <= 1e-6


@BOTH
@pytest.mark.parametrize("W,ff,E,top,shared,N", [(64, 40, 6, 2, 24, 37), (100, 30, 5, 5, None, 9), (128, 16, 70, 1, 64, 50),
                                                 (128, 64, 4, 2, 64, 700), (48, 32, 3, 2, None, 1)])
def test_routed_experts(dtype, W, ff, E, top, shared, N):
    """Experts without a gate (squared relu) behind the softmax-first router, a shared expert of another width; few
    tokens (a product per token and expert) and many (the grouped tiled product)."""
    rt = runtime(dtype)
    mlp = MM._moe(E, top, ff, shared)
    cfg = {"vocab": 4, "width": W, "max_positions": 4, "norm": {"eps": EPS},
           "layers": [{"type": "attention", "mixer": MM._attn(1, 1, 8, 8, 1.0), "mlp": mlp}]}
    w = {k[len("l0.mlp."):]: v.double() for k, v in PM.random_weights(cfg, E).items() if k.startswith("l0.mlp.")}
    part, w = build("feed_forward", "routed_experts", {
        "hidden_size": W, "intermediate_size": ff, "num_experts": E, "top": top, "gated": False,
        "activation": "relu_squared", "router": "softmax_top", "shared_ff": shared}, rt, tensors=w)
    x = _x(N, W, dtype, 3)
    margins = []
    want = PM.routed_ff(x.double(), w, "", mlp, margins=margins)
    sure = margins[0] > (CLOSE_CALL if dtype == "bfloat16" else 1e-3) if margins else torch.ones(N, dtype=torch.bool)
    got = dense(part.forward(x.to(DEV).to(rt.dtype), None), rt).float().cpu()
    tol = _tol(dtype, want[sure], lambda: PM.routed_ff(x.double(), w, "", mlp, round_to=torch.bfloat16)[sure])
    assert sure.any() and rel_err(got[sure].to(rt.dtype), want[sure]) <= tol


@BOTH
def test_dense_feed_forward_with_the_erf_gelu(dtype):
    rt = runtime(dtype)
    part, w = build("feed_forward", "dense", {"hidden_size": 72, "intermediate_size": 200, "activation": "gelu",
                                              "names": ("up", "down")}, rt, seed=2)
    x = _x(45, 72, dtype, 3, 2.0)
    want = PM.small_ff(x.double(), w["up"], w["down"], PM.gelu_erf)
    got = dense(part.forward(x.to(DEV).to(rt.dtype), None), rt)
    assert rel_err(got, want) <= PART_TOL[dtype]
    tanh_form = PM.small_ff(x.double(), w["up"], w["down"], lambda z: 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3))))
    if dtype == "float32":
        assert rel_err(got, tanh_form) > 10 * PART_TOL[dtype]           # the other gelu is held apart


# ------------------------------------------------------------------------------------ the mixers alone
GLA_CASES = [(MM._gla(2, 16, 32, 8.0, 8), 64, 75), (MM._gla(3, 10, 24, 1.0, 3), 100, 50), (MM._gla(4, 64, 64, 4.0, 16), 128, 150),
             (MM._gla(1, 40, 16, 30.0, 5), 48, 90), (MM._gla(2, 128, 128, 16.0, 16), 64, 200), (MM._gla(5, 16, 16, 2.0, 7), 80, 21)]


@BOTH
@pytest.mark.parametrize("m,W,T", GLA_CASES)
def test_gated_linear_attention_alone(dtype, m, W, T):
    """The mixer over a state slot against the plain recurrence: whole, token by token, and in portions with single
    tokens and pairs between them; the slots hold what an earlier request left."""
    rt = runtime(dtype)
    mixer, w = build("mixer", "gla", _gla_params(m, W), rt, tensors=_mixer_weights("gla", m, W, T))
    x = _x(T, W, dtype, 13)
    want = PM.gla_mixer(x.double(), w, "", m, EPS)
    tol = _tol(dtype, want, lambda: PM.gla_mixer(x.double(), w, "", m, EPS, round_to=torch.bfloat16))
    cuts_list = [[T], [1] * T, [T - 14, 1, 1, 2, 1, 3, 6], [2, 2, 3, T - 7]]
    if T >= 140:
        cuts_list.append([70, 64, T - 134])
    for cuts in cuts_list:
        steps = Steps([(None, mixer.state_spec())], rt, slots=3)
        for pool in steps.cache.state:
            pool.fill_(3.0)                                     # what an earlier request left in the slots
        got = _run_mixer(mixer, steps, x, cuts, rt)
        assert rel_err(got.to(rt.dtype), want) <= tol, cuts[:3]


@BOTH
@pytest.mark.parametrize("nh,dim,vdim,tau", [(2, 16, 32, 8.0), (3, 10, 24, 1.0), (1, 128, 128, 16.0), (2, 40, 16, 0.25)])
def test_the_recurrence_in_tiles_against_the_recurrence_token_after_token(dtype, nh, dim, vdim, tau):
    """Requests of 1 to 300 rows whose ends fall on, before and behind the edges of the tiles, through slots out of
    order that hold earlier states, the tiles listed in any order: the tiles side by side give the rows and the final states of the walk token after
    token; with tau 0.25 the decays of a tile multiply to zero and nothing overflows."""
    from infernum_amd.kernels import api as K
    rt = runtime(dtype)
    g = torch.Generator().manual_seed(nh * dim)
    lens = [63, 64, 65, 1, 128, 129, 300, 2]
    N, B = sum(lens), len(lens)
    row = 2 * nh * dim + nh * vdim
    proj = torch.randn(N, row, generator=g).to(DEV).to(rt.dtype)
    z = (torch.randn(N, nh * dim, generator=g) * 3).to(DEV)
    zb = torch.randn(nh * dim, generator=g).to(DEV)
    floats = K.gla_state_floats(nh, dim, vdim)
    slots = torch.tensor([5, 0, 7, 2, 9, 1, 3, 8], dtype=torch.int32, device=DEV)
    state0 = torch.randn(10, floats, generator=g).to(DEV)
    starts = torch.tensor([sum(lens[:i]) for i in range(B + 1)], dtype=torch.int32, device=DEV)
    tiles = [(b, f) for b, n in enumerate(lens) for f in range(0, n, K.PREFILL_TILE_ROWS)]
    tiles = torch.tensor([tiles[i] for i in torch.randperm(len(tiles), generator=g).tolist()], dtype=torch.int32).to(DEV)
    want, got = torch.empty((N, nh * vdim), device=DEV), torch.full((N, nh * vdim), 7.0, device=DEV)
    s_want, s_got = state0.clone(), state0.clone()
    K.gla_scan(proj, 0, nh * dim, 2 * nh * dim, z, zb, tau, dim ** -0.5, s_want, want, starts, slots, nh, dim, vdim)
    K.gla_chunked(proj, 0, nh * dim, 2 * nh * dim, z, zb, tau, dim ** -0.5, s_got, got, starts, slots, tiles,
                  tiles.shape[0], 0, nh, dim, vdim)
    assert torch.isfinite(want).all() and torch.isfinite(s_want).all()
    assert rel_err(got, want.cpu()) <= 2e-5
    assert rel_err(s_got, s_want.cpu()) <= 2e-5
    assert torch.equal(s_got[4], state0[4]) and torch.equal(s_got[6], state0[6])          # slots of no request


@BOTH
def test_requests_of_unequal_length_side_by_side_in_the_recurrence(dtype):
    """Three requests in one step, then again with other lengths, through slots out of order, against each alone."""
    rt = runtime(dtype)
    m, W = MM._gla(2, 64, 64, 8.0, 8), 64
    mixer, w = build("mixer", "gla", _gla_params(m, W), rt, tensors=_mixer_weights("gla", m, W, 4))
    lens = [(130, 1, 70), (1, 66, 3), (1, 1, 1)]
    xs = [_x(sum(l[i] for l in lens), W, dtype, 30 + i) for i in range(3)]
    want = [PM.gla_mixer(x.double(), w, "", m, EPS) for x in xs]
    tol = max(_tol(dtype, want[i], lambda i=i: PM.gla_mixer(xs[i].double(), w, "", m, EPS, round_to=torch.bfloat16)) for i in range(3))
    steps = Steps([(None, mixer.state_spec())], rt, slots=4)
    ctx, packed = steps.begin([("warm", 5)])                    # takes slot 0 first, so the three sit in 1..3
    steps.end(packed)
    got, done = [[], [], []], [0, 0, 0]
    for step in lens:
        order = sorted(range(3), key=lambda i: step[i] != 1)    # single tokens come first in a step's rows
        ctx, packed = steps.begin([(f"r{i}", step[i]) for i in order])
        rows = torch.cat([xs[i][done[i]:done[i] + step[i]] for i in order])
        out = dense(mixer.forward(rows.to(DEV).to(rt.dtype), ctx, steps.views[0]), rt).float().cpu()
        steps.end(packed)
        p = 0
        for i in order:
            got[i].append(out[p:p + step[i]])
            p += step[i]
            done[i] += step[i]
    for i in range(3):
        assert rel_err(torch.cat(got[i]).to(rt.dtype), want[i]) <= tol, i


@BOTH
def test_a_state_that_reaches_hundreds_of_tokens_back(dtype):
    """The heads forget slowly (their decays' logits are large: a token's weight halves after some thousand places in
    one head and after some hundred in the other) and token 3's input is large: 600 tokens later the output still
    carries it, in a prompt, in the portion after it, and in tokens decoded one by one."""
    rt = runtime(dtype)
    m, W, T = MM._gla(2, 16, 32, 2.0, 4), 32, 640
    w = _mixer_weights("gla", m, W, 2)
    w["a2"] = torch.zeros_like(w["a2"])
    w["a2.b"] = torch.cat([torch.full((16,), 9.0), torch.full((16,), 5.0)]).double()
    mixer, w = build("mixer", "gla", _gla_params(m, W), rt, tensors=w)
    x = _x(T, W, dtype, 5, 0.5)
    x[3] *= 8.0
    if dtype == "bfloat16":
        x = x.to(torch.bfloat16).float()
    want = PM.gla_mixer(x.double(), w, "", m, EPS)
    x0 = x.clone()
    x0[3] = 0.0
    tol = _tol(dtype, want, lambda: PM.gla_mixer(x.double(), w, "", m, EPS, round_to=torch.bfloat16))
    shows = (want[-8:] - PM.gla_mixer(x0.double(), w, "", m, EPS)[-8:]).abs().max() / want.pow(2).mean().sqrt()
    assert shows > 5 * tol, (shows, tol)
    for cuts in ([T], [300, T - 305] + [1] * 5, [3, 1, 200, T - 204]):
        steps = Steps([(None, mixer.state_spec())], rt, slots=2)
        got = _run_mixer(mixer, steps, x, cuts, rt)
        assert rel_err(got.to(rt.dtype), want) <= tol, cuts[:2]


ATT_CASES = [(MM._attn(4, 2, 16, 32, 0.25, (0.5, 16)), 64, 75), (MM._attn(5, None, 26, 10, 0.3), 100, 50),
             (MM._attn(20, 1, 32, 64, 0.2, (0.1, 1)), 128, 130), (MM._attn(3, 3, 48, 16, 0.15, (1.0, 100)), 48, 140),
             (MM._attn(8, 2, 96, 32, 0.1, (0.25, 7)), 64, 90), (MM._attn(2, 1, 128, 128, 0.09), 64, 200)]


@BOTH
@pytest.mark.parametrize("m,W,T", ATT_CASES)
@pytest.mark.parametrize("ps", [4, 16])
def test_sigmoid_attention_alone(dtype, m, W, T, ps):
    """The mixer over a paged cache against the plain form: whole, and in portions with single tokens between them
    that cut pages and the steps of the queries' factor; freed pages hold NaN."""
    rt = runtime(dtype)
    mixer, w = build("mixer", "sigmoid_attention", _att_params(m, W), rt, tensors=_mixer_weights("attention", m, W, T))
    x = _x(T, W, dtype, 8)
    want = PM.attention_mixer(x.double(), w, "", m, EPS)
    tol = _tol(dtype, want, lambda: PM.attention_mixer(x.double(), w, "", m, EPS, round_to=torch.bfloat16))
    for cuts in ([T], [T - 9, 1, 1, 2, 1, 3, 1], [1] * 6 + [T - 6], [2, 2, 17, T - 21]):
        steps = Steps([(mixer.cache_spec(), None)], rt, page_size=ps, num_pages=256 // ps, poison=True)
        got = _run_mixer(mixer, steps, x, cuts, rt)
        assert rel_err(got.to(rt.dtype), want) <= tol, cuts[:3]


@pytest.mark.parametrize("nh,nkv,dim,vdim,ps", [(4, 2, 16, 32, 4), (20, 1, 32, 64, 12), (3, 3, 48, 16, 16), (8, 2, 128, 64, 8),
                                                (2, 1, 128, 128, 20)])
def test_sigmoid_attention_on_the_matrix_cores_against_the_plain_kernel(nh, nkv, dim, vdim, ps):
    """The kernels for single tokens (whole, and with the keys cut into 2, 5 and 64 parts) and for portions of
    prompts (rows of 1 to 150 behind 0 to 130 keys) give what the plain kernel gives on the same pages, of sizes that
    are and are not powers of two; places of the pages that no request holds are NaN."""
    from infernum_amd.kernels import api as K
    g = torch.Generator().manual_seed(nh * dim + ps)
    lens = [1, 2, 17, 64, 65, 200, 333]
    per = max(-(-n // ps) for n in lens)
    P = len(lens) * per + 3
    perm = torch.randperm(P, generator=g).tolist()
    bt = torch.full((len(lens), per), -1, dtype=torch.int32)
    k = torch.full((P, nkv, ps, dim), float("nan"))
    v = torch.full((P, nkv, vdim, ps), float("nan"))
    for b, n in enumerate(lens):
        for i in range(-(-n // ps)):
            page = perm.pop()
            bt[b, i] = page
            m = min(ps, n - i * ps)
            k[page, :, :m] = torch.randn(nkv, m, dim, generator=g)
            v[page, :, :, :m] = torch.randn(nkv, vdim, m, generator=g)
    k, v, bt = k.to(DEV).to(torch.bfloat16), v.to(DEV).to(torch.bfloat16), bt.to(DEV)
    r1, r2, pb = (torch.rand(nh, generator=g) * 0.8 + 0.2).to(DEV), (torch.rand(nh, generator=g) * 0.45 + 0.05).to(DEV), \
        (-1 - 2 * torch.rand(nh, generator=g)).to(DEV)
    scale = 0.5 / math.sqrt(dim)

    def rows(N):
        q = torch.randn(N, nh * dim + 8, generator=g).to(DEV).to(torch.bfloat16)[:, :nh * dim]
        gate = torch.randn(N, nh + 3, generator=g).to(DEV).to(torch.bfloat16)[:, 3:]
        return q, gate, torch.empty((N, nh * vdim), dtype=torch.bfloat16, device=DEV), \
            torch.full((N, nh * vdim), 7.0, dtype=torch.bfloat16, device=DEV)
    # single tokens: the last place of every request
    B = len(lens)
    q, gate, want, got = rows(B)
    pos, seq = torch.tensor([n - 1 for n in lens], dtype=torch.int32, device=DEV), torch.arange(B, dtype=torch.int32, device=DEV)
    want = want.float()
    k32, v32 = k.float(), v.float()                          # the plain kernel on the same values, in 32-bit throughout
    K.sigattn_generic(q.float(), k32, v32, gate.float(), want, seq, pos, bt, r1, r2, pb, nh, nkv, dim, vdim, scale)
    assert torch.isfinite(want).all()
    for parts in (1, 2, 5, 64, None):
        got.fill_(7.0)
        K.sigattn_decode(q, k, v, gate, got, pos, bt, r1, r2, pb, nh, nkv, dim, vdim, scale, max(lens), parts)
        assert rel_err(got, want.float().cpu()) <= PART_TOL["bfloat16"], parts
    # portions: the last rows of every request, of many lengths
    qlens = [1, 2, 16, 64, 65, 70, 150]
    ctx = [n - m for n, m in zip(lens, qlens)]
    starts = [0]
    for m in qlens:
        starts.append(starts[-1] + m)
    q, gate, want, got = rows(starts[-1])
    seq = torch.cat([torch.full((m,), b, dtype=torch.int32) for b, m in enumerate(qlens)]).to(DEV)
    pos = torch.cat([torch.arange(c, c + m, dtype=torch.int32) for c, m in zip(ctx, qlens)]).to(DEV)
    tiles = torch.tensor([(b, f) for b, m in enumerate(qlens) for f in range(0, m, K.PREFILL_TILE_ROWS)], dtype=torch.int32).to(DEV)
    want = want.float()
    K.sigattn_generic(q.float(), k32, v32, gate.float(), want, seq, pos, bt, r1, r2, pb, nh, nkv, dim, vdim, scale)
    K.sigattn_prefill(q, k, v, gate, got, torch.tensor(starts, dtype=torch.int32, device=DEV),
                      torch.tensor(ctx, dtype=torch.int32, device=DEV), bt, tiles, tiles.shape[0], r1, r2, pb, nh, nkv, dim,
                      vdim, scale)
    assert torch.isfinite(want).all() and rel_err(got, want.float().cpu()) <= PART_TOL["bfloat16"]
    # a key that is needed and has no page: NaN in its request's rows, never a stray read
    bt[5, 1] = -1
    K.sigattn_decode(q[:B], k, v, gate[:B], got[:B], torch.tensor([n - 1 for n in lens], dtype=torch.int32, device=DEV), bt, r1,
                     r2, pb, nh, nkv, dim, vdim, scale, max(lens), 1)
    assert torch.isnan(got[5]).all() and torch.isfinite(got[:5]).all() and torch.isfinite(got[6]).all()


def _standing_out(dtype, T, star, first):
    """A mixer (two heads over one key head of 128, values of 32) and inputs in which every query from row ``first`` on
    points at token ``star``'s key: wherever that key is visible its weight is near one, and every other key's is
    near zero (a low number b on every score), so the output is the star's value or nothing.  The keys come from a
    projection that does not see the direction u; the queries see u alone and answer it with the star's key."""
    rt = runtime(dtype)
    W, d = 48, 128
    m = MM._attn(2, 1, d, 32, 0.3)
    w = _mixer_weights("attention", m, W, 1)
    g = torch.Generator().manual_seed(4)
    u = torch.randn(W, generator=g).double()
    u /= u.norm()
    w["k"] = (w["k"] - (w["k"] @ u)[:, None] * u[None, :]).to(torch.bfloat16).double()
    w["k.b"] = torch.zeros(d, dtype=torch.float64)        # a bias would be a part that all keys share with the star's
    x = _x(T, W, dtype, 3, 1.0).double()
    x = x - (x @ u)[:, None] * u[None, :]
    k = PM.rms_norm(x @ w["k"].t() + w["k.b"], w["k.norm"], EPS)
    w["q"] = torch.cat([torch.outer(k[star], u)] * 2).to(torch.bfloat16).double()
    w["q.b"] = (0.3 * torch.randn(2 * d, generator=g)).to(torch.bfloat16).double()
    w["q.norm"] = torch.ones(2 * d, dtype=torch.float64)
    w["pb"] = torch.full((2,), -26.0, dtype=torch.float64)
    x[first:] += 4.0 * u
    x = x.float()
    if dtype == "bfloat16":
        x = x.to(torch.bfloat16).float()
    mixer, w = build("mixer", "sigmoid_attention", _att_params(m, W), rt, tensors=w)
    return rt, mixer, w, m, x


@BOTH
@pytest.mark.parametrize("star", [2, 7, 8, 11, 12])
def test_a_key_that_stands_out_at_the_causal_edge_and_at_page_borders(dtype, star):
    """Rows before the star's own point at its key and must not see it; the star's row sees it at distance zero; the
    star is a page's last place, its first, or inside one (pages of 4).  Whole, with the rows around the edge decoded
    one by one, with a portion that begins at the star, and in pairs."""
    T = 30
    rt, mixer, w, m, x = _standing_out(dtype, T, star, max(star - 2, 0))
    want = PM.attention_mixer(x.double(), w, "", m, EPS)
    rms = want.pow(2).mean().sqrt()
    tol = _tol(dtype, want, lambda: PM.attention_mixer(x.double(), w, "", m, EPS, round_to=torch.bfloat16))
    assert want[:star].abs().max() < 1e-2 * rms and want[star].abs().max() > 0.3 * rms     # nothing, then the value
    for cuts in ([T], [star - 1] + [1] * 4 + [T - star - 3], [star, T - star], [star + 1, T - star - 1], [2] * (T // 2)):
        steps = Steps([(mixer.cache_spec(), None)], rt, page_size=4, num_pages=16, poison=True)
        got = _run_mixer(mixer, steps, x, [c for c in cuts if c], rt)
        assert rel_err(got.to(rt.dtype), want) <= tol, cuts[:2]


@BOTH
def test_a_far_key_among_hundreds(dtype):
    """A key 600 places back that stands out must still be seen, through the distance term: in a prompt, in the
    portion after it, and by tokens decoded one by one."""
    T, star = 640, 3
    rt, mixer, w, m, x = _standing_out(dtype, T, star, 1)
    want = PM.attention_mixer(x.double(), w, "", m, EPS)
    other = x.clone()
    other[star] = _x(1, x.shape[1], dtype, 77)[0]                     # another token in its place: nothing stands out
    without = PM.attention_mixer(other.double(), w, "", m, EPS)
    tol = _tol(dtype, want, lambda: PM.attention_mixer(x.double(), w, "", m, EPS, round_to=torch.bfloat16))
    assert (want[-1] - without[-1]).abs().max() > 10 * tol * want.pow(2).mean().sqrt()
    for cuts in ([T], [300, 209, 1, 1, 1, 1, 1, T - 514], [3, 1, T - 10] + [1] * 6):
        steps = Steps([(mixer.cache_spec(), None)], rt, page_size=4, num_pages=192, poison=True)
        got = _run_mixer(mixer, steps, x, cuts, rt)
        assert rel_err(got.to(rt.dtype), want) <= tol, cuts[:2]


# ------------------------------------------------------------------------------------ the engine
class _Ref:
    """Plain logits of a request and which of its places no close call of a router reaches (bool [T])."""

    def __init__(self, logits, sure):
        self.logits, self.sure = logits, sure


def _plain(cfg, w, toks):
    margins = []
    logits = PM.forward(cfg, w, toks, margins=margins)
    routed = [i for i, l in enumerate(cfg["layers"]) if l.get("mlp") and l["mlp"]["kind"] == "moe"
              and l["mlp"]["router"]["top"] < l["mlp"]["router"]["experts"]]
    close = torch.zeros(len(toks), dtype=torch.bool)
    for i, mg in zip(routed, margins):
        c = mg < CLOSE_CALL
        # a close call moves its own place; below the last layer the state and the keys carry it to every later one
        close |= c if i == len(cfg["layers"]) - 1 else torch.cumsum(c.int(), 0) > 0
    return _Ref(logits, ~close)


def _requests(cfg, w, lengths, seed):
    """Requests of these lengths; of a few candidates each, the one whose routers stay sure of their experts longest."""
    reqs, refs = {}, {}
    for i, n in enumerate(lengths):
        best = None
        for attempt in range(4):
            toks = TT.make_requests(cfg["vocab"], (n,), seed=seed + 100 * i + attempt)["r0"]
            ref = _plain(cfg, w, toks)
            if best is None or int(ref.sure.sum()) > int(best[1].sure.sum()):
                best = (toks, ref)
            if bool(ref.sure.all()):
                break
        reqs[f"r{i}"], refs[f"r{i}"] = best
    return reqs, refs


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for name in NAMES:
        d = str(tmp_path_factory.mktemp(name))
        cfg, w = MM.write_model(name, d)
        reqs, ref = _requests(cfg, w, LENGTHS[name], 11)
        mreqs, mref = _requests(cfg, w, MIXED[name], 23)
        cost = 0.0
        for group, refs in ((reqs, ref), (mreqs, mref)):
            for r, t in group.items():
                if refs[r].sure.any():
                    rounded = PM.forward(cfg, w, t, round_to=torch.bfloat16)
                    diff = (rounded - refs[r].logits)[refs[r].sure].abs().max().item()
                    cost = max(cost, diff / refs[r].logits.pow(2).mean().sqrt().item())
        BF16_TOL[name] = max(TOL["bfloat16"], 3.0 * cost)
        print(f"{name}: rounding alone costs {cost:.2e} of the logits' RMS; sure places "
              f"{[(len(t), int(ref[r].sure.sum())) for r, t in reqs.items()]} "
              f"{[(len(t), int(mref[r].sure.sum())) for r, t in mreqs.items()]}")
        out[name] = (d, cfg, w, reqs, ref, mreqs, mref)
    return out


def _engine(model_dir, dtype, page_size, num_pages, slots=8, **kw):
    from infernum_amd import CacheConfig, Engine
    return Engine.from_pretrained(model_dir, dtype=dtype, **kw,
                                  cache_config=CacheConfig(page_size=page_size, num_pages=num_pages,
                                                           num_state_slots=slots, poison_freed_pages=True))


def _check(got, ref, dtype, what, name=None):
    tol = BF16_TOL.get(name, TOL[dtype]) if dtype == "bfloat16" else TOL[dtype]
    if not isinstance(next(iter(ref.values())), _Ref):
        ref = {r: _Ref(t, torch.ones(t.shape[0], dtype=torch.bool)) for r, t in ref.items()}
    assert len(got) == sum(v.logits.shape[0] for v in ref.values()) and all(torch.isfinite(t).all() for t in got.values())
    if dtype == "bfloat16":
        got = {(r, p): t for (r, p), t in got.items() if ref[r].sure[p]}
        assert len(got) >= 10, "too few places are sure of their experts"
    ref = {r: v.logits for r, v in ref.items()}
    worst, rms, where = TT.error_against(got, ref, every_place=dtype != "bfloat16")
    print(f"{what}: max|diff| = {worst:.3e}, rms of logits = {rms:.3e}, ratio {worst / rms:.2e} at {where} over {len(got)} places")
    assert worst == worst, f"{what}: NaN in the logits at {where}"
    assert worst <= tol * rms, f"{what}: max|diff| {worst:.3e} > {tol} * rms {rms:.3e} at {where}"


@BOTH
@pytest.mark.parametrize("name", NAMES)
def test_layers_one_by_one(models, name, dtype):
    """The logits of the models made of the first k layers (the same tensors), k = 1, 2, ...: a layer that differs
    shows at its own k."""
    import shutil
    from infernum_amd.engine import StepEntry
    d, cfg, w, reqs, ref, *_ = models[name]
    toks = reqs["r2"]
    for k in range(1, len(cfg["layers"]) + 1):
        sub, sd = dict(cfg, layers=cfg["layers"][:k]), d + f"_first{k}"
        keep = {n: t for n, t in w.items() if not (n[0] == "l" and n[1].isdigit()) or int(n[1:n.index(".")]) < k}
        MM.write_model(sub, sd, weights=keep)
        eng = _engine(sd, dtype, PAGE[name], 64)
        logits = eng.step([StepEntry("a", toks, list(range(len(toks))))]).cpu()
        _check({("a", p): logits[p] for p in range(len(toks))}, {"a": _plain(sub, keep, toks)}, dtype,
               f"{name} {dtype} first {k} layers", name)
        shutil.rmtree(sd, ignore_errors=True)


@BOTH
@pytest.mark.parametrize("name", NAMES)
@pytest.mark.parametrize("how", ["whole", "tail", "portions", "one_by_one"])
def test_one_request_at_a_time(models, name, dtype, how):
    d, cfg, w, reqs, ref, *_ = models[name]
    eng = _engine(d, dtype, PAGE[name], 64)
    steps = {"whole": TT.trace_whole, "tail": lambda r: TT.trace_tail_one_by_one(r, 40), "portions": TT.trace_portions,
             "one_by_one": lambda r: TT.trace_tail_one_by_one(r, 10 ** 6)}[how](reqs)
    got = TT.run_steps(eng, steps)
    _check(got, ref, dtype, f"{name} {dtype} {how}", name)
    eng.cache.check()
    assert all(eng.cache.free_pages(g) == 64 for g in range(len(eng.cache.groups)))
    if eng.program is not None:
        eng.program.check_guards()
        assert eng.program.num_python_ops == 0             # every part wrote its own launches


@BOTH
@pytest.mark.parametrize("name", NAMES)
def test_mixed_batches_with_pages_and_slots_used_again(models, name, dtype):
    d, cfg, w, _, _, reqs, ref = models[name]
    prompt_len = {r: max(2, len(t) - 20 - 7 * i) for i, (r, t) in enumerate(reqs.items())}
    steps, max_tokens = TT.trace_mixed(reqs, prompt_len, seed=5)
    ps = PAGE[name]
    eng = _engine(d, dtype, ps, -(-max_tokens // ps), slots=4)      # four slots for up to four live of more requests
    assert sum(-(-len(t) // 64) * 64 for t in reqs.values()) > max_tokens   # the pool cannot hold them all: pages come back
    assert len(reqs) > 4
    got = TT.run_steps(eng, steps)
    _check(got, ref, dtype, f"{name} {dtype} mixed", name)
    eng.cache.check()
    if dtype == "float32":
        # the same rows from a batch and alone: equal but for the rounding of 32-bit sums taken in another order (the
        # recurrence adds up a prompt's portions tile by tile, and the tiles begin where the portions do)
        alone = TT.run_steps(_engine(d, dtype, ps, 64), TT.trace_whole(reqs))
        assert all(rel_err(got[k], alone[k].cpu()) <= 1e-5 for k in got)


@BOTH
@pytest.mark.parametrize("name", ["X1", "X4"])
def test_long_decoding(models, name, dtype):
    """A short prompt, then 150 tokens one by one: the state moves on 150 times, the queries' factor steps under
    decoded tokens, pages fill and begin; decode steps are replayed from graphs after the first two."""
    d, cfg, w, *_ = models[name]
    reqs, ref = _requests(cfg, w, (160,), 3)
    eng = _engine(d, dtype, 16, 12)
    got = TT.run_steps(eng, TT.trace_tail_one_by_one(reqs, 150))
    _check(got, ref, dtype, f"{name} {dtype} long decoding", name)
    assert eng.graph_replays > 100


def test_greedy_generation_through_the_scheduler(models):
    """Runtime.generate_batch (scheduler, portions, the sampler's argmax) against the plain model's greedy tokens,
    in 32-bit; prompts of unequal length, more requests than run at once."""
    from infernum_amd import BatchConfig, GenerateOptions, Runtime
    d, cfg, w, *_ = models["X1"]
    prompts = list(TT.make_requests(cfg["vocab"], (5, 31, 2, 18, 9), seed=9).values())
    rt = Runtime.from_pretrained(d, dtype="float32", batch_config=BatchConfig(block_size=16, num_blocks=24,
                                                                              max_batch_size=3, max_prefill_tokens=8,
                                                                              max_tokens_per_step=16, step_token_multiple=1))
    outs = rt.generate_batch(prompts, GenerateOptions(max_new_tokens=12))
    for p, got in zip(prompts, outs):
        toks = list(p)
        for _ in range(12):
            toks.append(int(PM.forward(cfg, w, toks)[-1].argmax()))
        assert list(got) == toks[len(p):], (p, got, toks[len(p):])


@BOTH
def test_trace_run_and_generate_programs(models, tmp_path, dtype):
    """bin/trace_run and bin/generate as a user starts them, on a Malinex folder whose configuration does not tell
    the width of the decays' middle: the model class comes from config.json; steps on standard input, logits in
    files; generated tokens on standard output."""
    import json
    import os
    import subprocess
    import sys
    import numpy as np
    _, cfg, w, _, _, reqs, ref = models["X3"]
    d = str(tmp_path / "model")
    MM.write_model("X3", d, with_rank=False)
    prompt_len = {r: max(2, len(t) - 12) for r, t in reqs.items()}
    steps, max_tokens = TT.trace_mixed(reqs, prompt_len, seed=4)
    out = tmp_path / "out"
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    proc = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", d, "--dtype", dtype,
                           "--out", str(out), "--max-tokens", str(max_tokens)],
                          input="".join(json.dumps(s) + "\n" for s in steps), text=True, capture_output=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-3000:]
    assert proc.stdout.split("\n")[:-1] == [f"done {s['step']}" for s in steps]
    pos, got = {}, {}
    for s in steps:
        n_want = sum(len(e["want"]) for e in s["entries"])
        arr = np.fromfile(out / f"{s['step']}.f32", dtype="<f4").reshape(n_want, cfg["vocab"])
        row = 0
        for e in s["entries"]:
            base = pos.get(e["id"], 0)
            for k in e["want"]:
                got[(e["id"], base + k)] = torch.from_numpy(arr[row].copy())
                row += 1
            pos[e["id"]] = base + len(e["tokens"])
    _check(got, ref, dtype, f"trace_run X3 {dtype} mixed", "X3")
    if dtype == "float32":
        prompt = reqs["r4"][:9]
        gen = subprocess.run([sys.executable, os.path.join(root, "bin", "generate"), "-m", d, "--prompt-ids",
                              ",".join(map(str, prompt)), "-n", "6", "--greedy", "--dtype", "float32"],
                             text=True, capture_output=True, timeout=600)
        assert gen.returncode == 0, gen.stderr[-3000:]
        toks = list(prompt)
        for _ in range(6):
            toks.append(int(PM.forward(cfg, w, toks)[-1].argmax()))
        assert " " + " ".join(map(str, toks[9:])) + "\n" in gen.stdout, gen.stdout[-2000:]
