"""The Sikazen decoder on the GPU against the plain implementation (plain_sikazen.py): each mechanism alone, then the
engine on small models of other sizes than any real one: whole prompts, the tail decoded token by token, portions
down to two tokens, mixed batches over pools so small that pages and state slots are used again (freed pages hold
NaN), a key that stands out just inside and just outside the window, in a block that is just seen and not yet seen,
far back among hundreds, a state that reaches hundreds of tokens back, long decoding from graphs, and greedy
generation through the runtime and its scheduler."""
import math

import pytest
import torch

import plain_sikazen as PS
import sikazen_models as SM
import trace_tools as TT
from part_harness import DEV, TOL as PART_TOL, Steps, build, dense, rel_err, runtime

pytestmark = pytest.mark.gpu
BOTH = pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
# largest |difference| of a logit as a fraction of the RMS of the plain logits
TOL = {"float32": 3e-5, "bfloat16": 6e-2}
NAMES = ["S1", "S2", "S3", "S4", "S5"]
LENGTHS = {"S1": (1, 7, 45, 83, 130), "S2": (3, 61, 33, 97), "S3": (9, 70, 121), "S4": (2, 17, 64, 150), "S5": (1, 64, 65, 140)}
MIXED = {"S1": (70, 131, 64, 150, 33, 97, 66, 81), "S2": (150, 165, 120, 190, 147), "S3": (129, 65, 90, 47, 72, 99),
         "S4": (70, 131, 64, 150, 33, 97), "S5": (150, 100, 64, 190, 129, 77)}
PAGE = {"S1": 16, "S2": 4, "S3": 8, "S4": 16, "S5": 12}
BF16_TOL, F32_TOL = {}, {}
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
    cfg = {"vocab": 4, "width": W, "norm": {"eps": EPS}, "layers": [{"type": kind, "mixer": m, "mlp": None}]}
    return {k[len("l0.mix."):]: v.double() for k, v in PS.random_weights(cfg, seed).items() if k.startswith("l0.mix.")}


def _rope(rot, head_dim, pairing):
    if not rot:
        return {"kind": "none"}
    factor = (rot.get("scaling") or {}).get("factor")
    return {"kind": "rope", "params": {"head_dim": head_dim, "theta": rot["base"], "rotary_dim": rot["dims"],
                                       "scaling": {"rope_type": "linear", "factor": factor} if factor else None,
                                       "pairing": pairing}}


def _att_params(m, W):
    mask = m.get("mask") or {}
    return {"hidden_size": W, "num_heads": m["heads"], "num_kv_heads": m["kv_heads"], "head_dim": m["dim"],
            "value_dim": m["vdim"], "scale": m["scale"], "position": _rope(m.get("rot"), m["dim"], "half"),
            "window": mask.get("size"), "pool": mask.get("pool"), "norm_eps": EPS}


def _lat_params(m, W):
    return {"hidden_size": W, "num_heads": m["heads"], "head_dim": m["dim"], "rot_dim": m["rot_dim"],
            "value_dim": m["vdim"], "rank": m["kv_rank"], "q_rank": m["q_rank"], "norm_eps": EPS, "scale": m["scale"],
            "position": _rope(m["rot"], m["rot_dim"] + m["kv_rank"], "neighbours"), "gate": False, "sink": True}


def _hgrn_params(m, W):
    return {"hidden_size": W, "num_heads": m["heads"], "head_dim": m["dim"], "value_dim": m["vdim"], "norm_eps": EPS}


def _steps_for(mixer, rt, page_size, num_pages, slots=4, poison=True):
    """A cache for one mixer: its pages or state and, where it keeps a second kind of thing, that too."""
    needs = [(mixer.cache_spec(), mixer.state_spec())]
    names = []
    for name, part in getattr(mixer, "cached_companions", lambda: {})().items():
        needs.append((part.cache_spec(), part.state_spec()))
        names.append(name)
    steps = Steps(needs, rt, page_size=page_size, num_pages=num_pages, slots=slots, poison=poison)
    steps.views[0].others = {n: steps.views[1 + i] for i, n in enumerate(names)}
    return steps


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


CUTS = lambda T: ([T], [1] * T, [T - 9] + [1] * 9, [2] * (T // 2) + [T % 2] * (T % 2), [7, 2, 13, 2, 3, T - 27])  # noqa: E731


# ------------------------------------------------------------------------------------ small kernels alone
@BOTH
@pytest.mark.parametrize("N,C,col,extra", [(1, 8, 0, 0), (37, 80, 5, 9), (200, 24, 0, 40), (3, 300, 2, 1)])
def test_rows_divided_by_their_root_mean_square(dtype, N, C, col, extra):
    from infernum_amd.kernels import api as K
    rt = runtime(dtype)
    x = _x(N, col + C + extra, dtype, 1, 3.0)
    w = (torch.rand(C, generator=torch.Generator().manual_seed(2)) + 0.5)
    got = K.rms_rows(x.to(DEV).to(rt.dtype), col, C, w.to(DEV), 1e-3)
    want = PS.unit_rms(x[:, col:col + C].double(), 1e-3) * w.double()
    assert rel_err(got, want) <= PART_TOL[dtype]
    got = K.rms_rows(x.to(DEV).to(rt.dtype), col, C, None, 1e-3)
    assert rel_err(got, PS.unit_rms(x[:, col:col + C].double(), 1e-3)) <= PART_TOL[dtype]


@BOTH
def test_token_input_alone(dtype):
    """A layer's part of the second table, the gate, the product, the norm and the add into the fp32 stream."""
    rt = runtime(dtype)
    W, V, dim, layers, layer = 40, 50, 6, 3, 1
    g = torch.Generator().manual_seed(4)
    table = torch.randn(V, dim * layers, generator=g)
    part, w = build("token_input", "gated_table", {"hidden_size": W, "vocab_size": V, "dim": dim, "column": layer * dim,
                                                   "columns": dim * layers, "eps": EPS, "table": "side.embed",
                                                   "names": ("embed", "gate", "proj", "norm")}, rt,
                    tensors={"embed": table}, seed=5)
    toks = torch.randint(0, V, (23,), generator=g)
    h = torch.randn(23, W, generator=g) * 2
    named = {"side.embed": w["embed"], f"l{layer}.side.gate": w["gate"], f"l{layer}.side.proj": w["proj"],
             f"l{layer}.side.norm": w["norm"]}
    want = h.double() + PS.token_side_input(h.double(), toks, named, layer, dim, EPS)
    rounded = h.double() + PS.token_side_input(h.double(), toks, named, layer, dim, EPS, round_to=torch.bfloat16)

    class Ctx:
        token_ids = toks.to(torch.int32).to(DEV)
    hd = h.to(DEV)
    part.forward(hd, Ctx)
    tol = PART_TOL[dtype] if dtype == "float32" else max(PART_TOL[dtype], 3 * rel_err(rounded.float(), want))
    assert rel_err(hd, want) <= tol


# ------------------------------------------------------------------------------------ the mixers alone
ATT_CASES = [(SM.S1["layers"][0]["mixer"], 64, 70), (SM.S2["layers"][0]["mixer"], 100, 45), (SM.S2["layers"][2]["mixer"], 100, 40),
             (SM.S3["layers"][0]["mixer"], 128, 33), (SM.S5["layers"][0]["mixer"], 48, 50), (SM.S5["layers"][1]["mixer"], 48, 90)]


@BOTH
@pytest.mark.parametrize("m,W,T", ATT_CASES)
@pytest.mark.parametrize("ps", [4, 16])
def test_pooled_window_attention_alone(dtype, m, W, T, ps):
    """Whole, token by token, a tail decoded, in pairs, in uneven portions: over pages of 4 and 16, so that blocks
    straddle pages, and with the pages that the window and the open block have left given back and poisoned."""
    rt = runtime(dtype)
    mixer, w = build("mixer", "pooled_window_attention", _att_params(m, W), rt, tensors=_mixer_weights("attention", m, W, 3))
    x = _x(T, W, dtype, 7)
    want = PS.attention_mixer(x.double(), w, "", m, EPS)
    tol = _tol(dtype, want, lambda: PS.attention_mixer(x.double(), w, "", m, EPS, round_to=torch.bfloat16))
    for cuts in CUTS(T):
        steps = _steps_for(mixer, rt, ps, 2 * (-(-T // ps)) + 2)
        got = _run_mixer(mixer, steps, x, cuts, rt)
        assert rel_err(got.to(rt.dtype), want) <= tol, cuts[:3]
        if m.get("mask"):       # the window's group holds what the window and the open block reach, no more
            reach = max(m["mask"]["size"], m["mask"].get("pool") or 0)
            assert len([p for p in steps.cache.block_table(0, "a").pages if p >= 0]) <= -(-reach // ps) + 1


def _standing_out(dtype, T, star, size, pool, d=16, scale=3.0):
    """A mixer of one head whose queries all point one way, and a token whose key alone points that way too; the
    other keys are orthogonal to it.  The star's value is 5 in the first place, the others' are 0, and the output
    projection passes that place on: a row shows 5 times the weight it gives the star, as a key of its own (about 5),
    as a member of a block (about 5 / pool), or not at all."""
    W = 8
    rt = runtime(dtype)
    m = {"heads": 1, "kv_heads": 1, "dim": d, "vdim": 16, "scale": scale, "mask": {"size": size, "pool": pool}}
    w = {n: torch.zeros(s, dtype=torch.float64) for n, s in (("q", (d, W)), ("q.b", (d,)), ("k", (d, W)), ("k.b", (d,)),
                                                             ("v", (16, W)), ("v.b", (16,)), ("o", (W, 16)))}
    w["q"][0, 0] = 1.0          # q = (x0, 0, ...): with x0 = 1 a unit vector of length sqrt(d) along the first place
    w["k"][0, 1] = 1.0          # k = (x1, x2, 0, ...)
    w["k"][1, 2] = 1.0
    w["v"][0, 3] = 1.0
    w["o"][0, 0] = 1.0
    x = torch.zeros(T, W)
    x[:, 0], x[:, 2] = 1.0, 1.0
    x[star, 1], x[star, 2], x[star, 3] = 1.0, 0.0, 5.0
    mixer, w = build("mixer", "pooled_window_attention", _att_params(m, W), rt, tensors=w)
    return rt, mixer, w, m, x


@BOTH
@pytest.mark.parametrize("star,size,pool", [(9, 7, 4), (8, 7, 4), (11, 5, 6), (3, 16, 4), (12, 4, 9), (15, 1, 1)])
def test_a_key_that_stands_out_at_the_windows_edge_and_at_a_blocks(dtype, star, size, pool):
    """Rows star .. star + size - 1 see the star as a key of its own; the rows after them do not see it until its
    block is whole and lies before the window, and from then on they see it in the block's mean.  Whole, decoded
    across both edges, in portions that begin at an edge, in pairs; pages of 4."""
    T = 48
    rt, mixer, w, m, x = _standing_out(dtype, T, star, size, pool)
    want = PS.attention_mixer(x.double(), w, "", m, EPS)
    tol = _tol(dtype, want, lambda: PS.attention_mixer(x.double(), w, "", m, EPS, round_to=torch.bfloat16))
    last_in = star + size - 1                                   # the last row whose window holds the star
    first_block = (star // pool) * pool + pool - 1 + size       # the first row that sees the star's block
    col = want[:, 0]
    assert col[:star].abs().max() < 1e-3 and col[star:last_in + 1].min() > 4.0
    if first_block > last_in + 1:
        assert col[last_in + 1:first_block].abs().max() < 1e-3, "between the window and the block the star is not seen"
    assert col[first_block:].min() > 2.5 / pool and col[first_block:].max() < 5.5 / pool + 1e-3
    # (blocks of one position are their position's key and value: what leaves the window is seen on, the same)
    for one_off in ({"size": size + 1, "pool": pool}, {"size": max(size - 1, 1), "pool": pool}) if pool > 1 else ():
        other = PS.attention_mixer(x.double(), w, "", dict(m, mask=one_off), EPS)
        assert (other[:, 0] - col).abs().max() > 0.5 / pool       # a window one place off shows
    for cuts in ([T], [last_in] + [1] * 3 + [T - last_in - 3], [last_in + 1, T - last_in - 1],
                 [first_block - 1] + [1] * 3 + [T - first_block - 2], [first_block, T - first_block], [2] * (T // 2), [1] * T):
        steps = _steps_for(mixer, rt, 4, 16)
        got = _run_mixer(mixer, steps, x, [c for c in cuts if c > 0], rt)
        assert rel_err(got.to(rt.dtype), want) <= tol, cuts[:3]


@BOTH
def test_a_far_block_among_hundreds(dtype):
    """A star 600 places back is seen through its block's mean, in a prompt, in the portion after it, and by tokens
    decoded one by one, long after the pages of its own keys went back to the pool."""
    T, star, size, pool = 640, 5, 24, 8
    rt, mixer, w, m, x = _standing_out(dtype, T, star, size, pool)
    want = PS.attention_mixer(x.double(), w, "", m, EPS)
    assert want[-1, 0] > 2.5 / pool
    tol = _tol(dtype, want, lambda: PS.attention_mixer(x.double(), w, "", m, EPS, round_to=torch.bfloat16))
    for cuts in ([T], [300, 209, 1, 1, 1, 1, 1, T - 514], [3, 1, T - 10] + [1] * 6):
        steps = _steps_for(mixer, rt, 4, 176)
        got = _run_mixer(mixer, steps, x, cuts, rt)
        assert rel_err(got.to(rt.dtype), want) <= tol, cuts[:2]
        assert len([p for p in steps.cache.block_table(0, "a").pages if p >= 0]) <= 8


LAT_CASES = [(SM.S1["layers"][1]["mixer"], 64, 70), (SM.S2["layers"][1]["mixer"], 100, 45), (SM.S5["layers"][2]["mixer"], 48, 130)]


@BOTH
@pytest.mark.parametrize("m,W,T", LAT_CASES)
@pytest.mark.parametrize("ps", [4, 16])
def test_latent_attention_with_a_query_latent_and_sinks_alone(dtype, m, W, T, ps):
    rt = runtime(dtype)
    mixer, w = build("mixer", "latent_attention", _lat_params(m, W), rt, tensors=_mixer_weights("latent_attention", m, W, 3))
    x = _x(T, W, dtype, 8)
    want = PS.latent_attention_mixer(x.double(), w, "", m, EPS)
    tol = _tol(dtype, want, lambda: PS.latent_attention_mixer(x.double(), w, "", m, EPS, round_to=torch.bfloat16))
    # the sinks matter here: without them the rows differ by far more than the tolerance
    no_sink = PS.latent_attention_mixer(x.double(), dict(w, sink=torch.full_like(w["sink"], -1e9)), "", m, EPS)
    assert rel_err(no_sink.float(), want) > 0.1
    for cuts in CUTS(T):
        steps = _steps_for(mixer, rt, ps, -(-T // ps) + 1)
        got = _run_mixer(mixer, steps, x, cuts, rt)
        assert rel_err(got.to(rt.dtype), want) <= tol, cuts[:3]


@BOTH
def test_a_sink_that_takes_nearly_everything(dtype):
    """With a sink above every score the mixer's result shrinks to a fraction; with one far below it is the plain
    softmax's.  Both through prompts (the kernel for portions) and single tokens (the kernels for those, whose parts
    of the keys are joined where the sink is counted once)."""
    m, W, T = dict(SM.S5["layers"][2]["mixer"], heads=2), 48, 150
    rt = runtime(dtype)
    w = _mixer_weights("latent_attention", m, W, 3)
    x = _x(T, W, dtype, 9)
    for sink in (6.0, -30.0, 0.0):
        w["sink"] = torch.tensor([sink, sink / 2], dtype=torch.float64)
        mixer, wb = build("mixer", "latent_attention", _lat_params(m, W), rt, tensors=w)
        want = PS.latent_attention_mixer(x.double(), wb, "", m, EPS)
        tol = _tol(dtype, want, lambda: PS.latent_attention_mixer(x.double(), wb, "", m, EPS, round_to=torch.bfloat16))
        for cuts in ([T], [T - 40] + [1] * 40):
            steps = _steps_for(mixer, rt, 16, 12)
            got = _run_mixer(mixer, steps, x, cuts, rt)
            assert rel_err(got.to(rt.dtype), want) <= tol, (sink, cuts[:2])


@pytest.mark.parametrize("nh,nkv,d,ps,splits", [(4, 2, 64, 16, 1), (4, 2, 64, 16, 3), (16, 1, 112, 8, 2), (3, 3, 32, 4, 1)])
def test_sinks_in_the_matrix_core_kernels_against_the_plain_kernel(nh, nkv, d, ps, splits):
    from infernum_amd.kernels import api as K
    if not K.attention_mfma_available(d):
        pytest.skip("no matrix-core kernel for this head size")
    g = torch.Generator().manual_seed(5)
    lens = [70, 33, 129]
    B, MB = len(lens), -(-max(lens) // ps)
    num_pages = B * MB + 3
    kp = torch.randn(num_pages, nkv, ps, d, generator=g).to(torch.bfloat16).to(DEV)
    vp = torch.randn(num_pages, nkv, d, ps, generator=g).to(torch.bfloat16).to(DEV)
    perm = torch.randperm(num_pages, generator=g)[:B * MB].view(B, MB).to(torch.int32).to(DEV)
    sinks = (torch.randn(nh, generator=g) * 2 + 3).to(DEV)
    scale = 0.3 / math.sqrt(d) * 4
    # single tokens at every request's last place
    q = torch.randn(B, nh * d, generator=g).to(torch.bfloat16).to(DEV)
    pos = torch.tensor([n - 1 for n in lens], dtype=torch.int32, device=DEV)
    seq = torch.arange(B, dtype=torch.int32, device=DEV)
    want, got = torch.empty_like(q), torch.empty_like(q)
    K.attention_generic(q, kp, vp, want, seq, pos, perm, nh, nkv, d, scale, 0, sinks=sinks)
    K.attention_decode(q, kp, vp, got, pos, perm, nh, nkv, d, scale, 0, max(lens), num_splits=splits, sinks=sinks)
    assert rel_err(got, want.double().cpu()) <= 3e-2
    plain = torch.empty_like(q)
    K.attention_generic(q, kp, vp, plain, seq, pos, perm, nh, nkv, d, scale, 0)
    assert rel_err(plain, want.double().cpu()) > 5e-2                      # the sinks are felt
    # whole prompts
    N = sum(lens)
    q = torch.randn(N, nh * d, generator=g).to(torch.bfloat16).to(DEV)
    starts = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32, device=DEV)
    ctx = torch.zeros(B, dtype=torch.int32, device=DEV)
    seq = torch.cat([torch.full((n,), i, dtype=torch.int32) for i, n in enumerate(lens)]).to(DEV)
    pos = torch.cat([torch.arange(n, dtype=torch.int32) for n in lens]).to(DEV)
    tiles = torch.tensor([(s, r) for s, n in enumerate(lens) for r in range(0, n, K.PREFILL_TILE_ROWS)], dtype=torch.int32).to(DEV)
    want, got = torch.empty_like(q), torch.empty_like(q)
    K.attention_generic(q, kp, vp, want, seq, pos, perm, nh, nkv, d, scale, 0, sinks=sinks)
    K.attention_prefill(q, kp, vp, got, starts, ctx, perm, tiles, tiles.shape[0], nh, nkv, d, scale, 0, sinks=sinks)
    assert rel_err(got, want.double().cpu()) <= 3e-2


@pytest.mark.parametrize("nh,nkv,d,dv,ps,window,pool", [(4, 2, 16, 32, 4, 20, 6), (6, 2, 64, 64, 16, 40, 10), (20, 1, 32, 16, 8, 1, 1),
                                                        (3, 3, 48, 16, 12, 0, 0), (4, 2, 16, 16, 16, 33, 16), (2, 1, 128, 128, 16, 7, 9),
                                                        (17, 1, 16, 16, 4, 40, 5)])
def test_window_and_blocks_on_the_matrix_cores_against_the_plain_kernel(nh, nkv, d, dv, ps, window, pool):
    """Requests of unequal length with their pages in a shuffled order, NaN in every page that no request holds and in
    the pages of keys that have left every window; single tokens at each request's last place, and portions that
    begin anywhere, with and without sinks."""
    from infernum_amd.kernels import api as K
    g = torch.Generator().manual_seed(7)
    lens, starts_at = [70, 33, 129, 16, 200], [0, 20, 64, 15, 131]
    B, MB = len(lens), -(-max(lens) // ps)
    num_pages = B * MB + 5
    nan = float("nan")
    kp = torch.full((num_pages, nkv, ps, d), nan)
    vp = torch.full((num_pages, nkv, dv, ps), nan)
    E = K.wpa_pool_entries(ps, pool) if pool else 1
    pk, pv = torch.full((num_pages, nkv, E, d), nan), torch.full((num_pages, nkv, E, dv), nan)
    perm = torch.randperm(num_pages, generator=g)
    bt = torch.full((B, MB), -1, dtype=torch.int32)
    btp = torch.full((B, MB), -1, dtype=torch.int32)
    for b, n in enumerate(lens):
        reach = max(window, pool) if window else n
        for pg in range(-(-n // ps)):
            page = int(perm[b * MB + pg])
            btp[b, pg] = page
            if (pg + 1) * ps > n - reach - ps:              # pages that some query of the tests below still needs
                bt[b, pg] = page
                kp[page] = torch.randn(nkv, ps, d, generator=g)
                vp[page] = torch.randn(nkv, dv, ps, generator=g)
            pk[page] = torch.randn(nkv, E, d, generator=g)
            pv[page] = torch.randn(nkv, E, dv, generator=g)
    dev = lambda t: t.to(torch.bfloat16).to(DEV) if t.dtype.is_floating_point else t.to(DEV)   # noqa: E731
    kp, vp, pk, pv, bt, btp = map(dev, (kp, vp, pk, pv, bt, btp))
    scale = 2.0 / math.sqrt(d)
    for sinks in (None, (torch.randn(nh, generator=g) * 2 + 1).to(DEV)):
        # single tokens
        q = dev(torch.randn(B, nh * d, generator=g))
        pos = torch.tensor([n - 1 for n in lens], dtype=torch.int32, device=DEV)
        seq = torch.arange(B, dtype=torch.int32, device=DEV)
        want, got = torch.empty((B, nh * dv), dtype=torch.bfloat16, device=DEV), torch.empty((B, nh * dv), dtype=torch.bfloat16, device=DEV)
        K.wpa_attention(q, kp, vp, pk, pv, want, sinks, seq, pos, bt, btp, nh, nkv, scale, window, pool)
        K.wpa_decode(q, kp, vp, pk, pv, got, sinks, pos, bt, btp, nh, nkv, scale, window, pool)
        assert torch.isfinite(want.float()).all()
        assert rel_err(got, want.double().cpu()) <= 3e-2
        # portions: request b brings its rows from starts_at[b] on (what lies before is cached)
        news = [n - s0 for n, s0 in zip(lens, starts_at)]
        if window:          # the rows of a portion reach back from its first row: only portions whose keys have pages
            news = [min(k, ps) for k in news]
            first = [n - k for n, k in zip(lens, news)]
        else:
            first = starts_at
        N = sum(news)
        q = dev(torch.randn(N, nh * d, generator=g))
        starts = torch.tensor([0] + list(torch.tensor(news).cumsum(0)), dtype=torch.int32, device=DEV)
        ctx = torch.tensor(first, dtype=torch.int32, device=DEV)
        seq = torch.cat([torch.full((k,), i, dtype=torch.int32) for i, k in enumerate(news)]).to(DEV)
        pos = torch.cat([torch.arange(f, f + k, dtype=torch.int32) for f, k in zip(first, news)]).to(DEV)
        tiles = torch.tensor([(s_, r) for s_, k in enumerate(news) for r in range(0, k, K.PREFILL_TILE_ROWS)], dtype=torch.int32).to(DEV)
        want, got = torch.empty((N, nh * dv), dtype=torch.bfloat16, device=DEV), torch.empty((N, nh * dv), dtype=torch.bfloat16, device=DEV)
        K.wpa_attention(q, kp, vp, pk, pv, want, sinks, seq, pos, bt, btp, nh, nkv, scale, window, pool)
        K.wpa_prefill(q, kp, vp, pk, pv, got, sinks, starts, ctx, bt, btp, tiles, tiles.shape[0], nh, nkv, scale, window, pool)
        assert torch.isfinite(want.float()).all()
        assert rel_err(got, want.double().cpu()) <= 3e-2


HGRN_CASES = [(SM.S1["layers"][2]["mixer"], 64, 150), (SM.S2["layers"][3]["mixer"], 100, 70), (SM.S3["layers"][1]["mixer"], 128, 131),
              (SM.S4["layers"][1]["mixer"], 80, 64)]


@BOTH
@pytest.mark.parametrize("m,W,T", HGRN_CASES)
def test_hgrn2_alone(dtype, m, W, T):
    """Whole (tiles of rows side by side), token by token (the walk), and mixtures of both: the state is carried."""
    rt = runtime(dtype)
    mixer, w = build("mixer", "hgrn2", _hgrn_params(m, W), rt, tensors=_mixer_weights("hgrn2", m, W, 3))
    x = _x(T, W, dtype, 10)
    want = PS.hgrn2_mixer(x.double(), w, "", m, EPS)
    tol = _tol(dtype, want, lambda: PS.hgrn2_mixer(x.double(), w, "", m, EPS, round_to=torch.bfloat16))
    steps = _steps_for(mixer, rt, 16, 4, slots=2)
    for i, cuts in enumerate(CUTS(T) + ([64, T - 64] if T > 64 else [T],)):
        # slots are used again: every request finds one that an earlier request left full
        got = _run_mixer(mixer, steps, x, [c for c in cuts if c > 0], rt, request=f"r{i}")
        steps.cache.release(f"r{i}")
        assert rel_err(got.to(rt.dtype), want) <= tol, cuts[:3]


@BOTH
def test_requests_of_unequal_length_side_by_side_in_the_recurrence(dtype):
    m, W = SM.S1["layers"][2]["mixer"], 64
    rt = runtime(dtype)
    mixer, w = build("mixer", "hgrn2", _hgrn_params(m, W), rt, tensors=_mixer_weights("hgrn2", m, W, 4))
    lens = {"a": 1, "b": 130, "c": 64, "d": 65, "e": 1, "f": 7}
    xs = {r: _x(n + 3, W, dtype, 20 + i) for i, (r, n) in enumerate(lens.items())}
    want = {r: PS.hgrn2_mixer(x.double(), w, "", m, EPS) for r, x in xs.items()}
    steps = _steps_for(mixer, rt, 16, 4, slots=6)
    got = {r: [] for r in lens}
    order = list(lens)
    for portion in (lambda r: lens[r], lambda r: 1, lambda r: 2):
        entries = [(r, portion(r)) for r in order if len(got[r]) == 0 or True]
        done = {r: sum(t.shape[0] for t in got[r]) for r in order}
        ctx, packed = steps.begin(entries)
        rows = torch.cat([xs[e.request][done[e.request]:done[e.request] + len(e.tokens)] for e in packed.batch])
        y = dense(mixer.forward(rows.to(DEV).to(rt.dtype), ctx, steps.views[0]), rt).float().cpu()
        steps.end(packed)
        at = 0
        for e in packed.batch:
            got[e.request].append(y[at:at + len(e.tokens)])
            at += len(e.tokens)
    tol = PART_TOL[dtype] if dtype == "float32" else 2 * PART_TOL[dtype]
    for r in lens:
        assert rel_err(torch.cat(got[r]).to(rt.dtype), want[r]) <= tol, r


@BOTH
def test_a_state_that_reaches_hundreds_of_tokens_back(dtype):
    """A head whose gate stays near one carries what token 3 wrote over 600 tokens and ten tiles, whole and decoded."""
    m, W, T = {"heads": 2, "dim": 16, "vdim": 16}, 32, 640
    rt = runtime(dtype)
    w = _mixer_weights("hgrn2", m, W, 5)
    w["lower"] = torch.full_like(w["lower"], 1.0 - 2.0 ** -8)         # (a bfloat16 number: the next one up is one)
    w["lower"][16:] = 0.5                                   # the second head forgets within a few tokens
    x = _x(T, W, dtype, 11, 0.2)
    x[3] = _x(1, W, dtype, 12, 6.0)[0]
    mixer, w = build("mixer", "hgrn2", _hgrn_params(m, W), rt, tensors=w)
    want = PS.hgrn2_mixer(x.double(), w, "", m, EPS)
    other = x.clone()
    other[3] = x[4]
    without = PS.hgrn2_mixer(other.double(), w, "", m, EPS)
    tol = _tol(dtype, want, lambda: PS.hgrn2_mixer(x.double(), w, "", m, EPS, round_to=torch.bfloat16))
    assert (want[-1] - without[-1]).abs().max() > 10 * tol * want.pow(2).mean().sqrt()
    for cuts in ([T], [300, 209, 1, 1, 1, 1, 1, T - 514], [3, 1, T - 10] + [1] * 6):
        steps = _steps_for(mixer, rt, 16, 4, slots=2)
        got = _run_mixer(mixer, steps, x, cuts, rt)
        assert rel_err(got.to(rt.dtype), want) <= tol, cuts[:2]


# ------------------------------------------------------------------------------------ the engine
def _requests(cfg, w, lengths, seed):
    reqs = TT.make_requests(cfg["vocab"], lengths, seed=seed)
    return reqs, {r: PS.forward(cfg, w, t) for r, t in reqs.items()}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for name in NAMES:
        d = str(tmp_path_factory.mktemp(name))
        cfg, w = SM.write_model(name, d)
        reqs, ref = _requests(cfg, w, LENGTHS[name], 11)
        mreqs, mref = _requests(cfg, w, MIXED[name], 23)
        cost = {torch.bfloat16: 0.0, torch.float32: 0.0}
        for group, refs in ((reqs, ref), (mreqs, mref)):
            for r, t in group.items():
                for to in cost:
                    rounded = PS.forward(cfg, w, t, round_to=to)
                    cost[to] = max(cost[to], (rounded - refs[r]).abs().max().item() / refs[r].pow(2).mean().sqrt().item())
        BF16_TOL[name] = max(TOL["bfloat16"], 3.0 * cost[torch.bfloat16])
        # in 32-bit the plain model rounds what is stored between kernels and none of the sums inside them: eight
        # times that (a place that multiplies every rounding fifty times over costs S3 2.6e-5 by it alone)
        F32_TOL[name] = max(TOL["float32"], 8.0 * cost[torch.float32])
        print(f"{name}: rounding alone costs {cost[torch.bfloat16]:.2e} (bfloat16) and {cost[torch.float32]:.2e} "
              f"(stored values in 32-bit) of the logits' RMS")
        out[name] = (d, cfg, w, reqs, ref, mreqs, mref)
    return out


def _engine(model_dir, dtype, page_size, num_pages, slots=8, **kw):
    from infernum_amd import CacheConfig, Engine
    return Engine.from_pretrained(model_dir, dtype=dtype, **kw,
                                  cache_config=CacheConfig(page_size=page_size, num_pages=num_pages,
                                                           num_state_slots=slots, poison_freed_pages=True))


def _check(got, ref, dtype, what, name=None):
    tol = (BF16_TOL if dtype == "bfloat16" else F32_TOL).get(name, TOL[dtype])
    assert all(torch.isfinite(t).all() for t in got.values())
    worst, rms, where = TT.error_against(got, ref)
    print(f"{what}: max|diff| = {worst:.3e}, rms of logits = {rms:.3e}, ratio {worst / rms:.2e} at {where} over {len(got)} places")
    assert worst == worst, f"{what}: NaN in the logits at {where}"
    assert worst <= tol * rms, f"{what}: max|diff| {worst:.3e} > {tol} * rms {rms:.3e} at {where}"


@BOTH
@pytest.mark.parametrize("name", NAMES)
def test_the_stream_after_every_layer_run(models, name, dtype):
    """The logits of the models made of the first k layers (the same tensors, the loop cut to what is left of it),
    k = 1, 2, ...: a layer that differs shows at its own k."""
    import copy
    import shutil
    from infernum_amd.engine import StepEntry
    d, cfg, w, reqs, ref, *_ = models[name]
    toks = reqs["r2"]
    for k in range(1, len(cfg["layers"]) + 1):
        sub = copy.deepcopy(cfg)
        sub["layers"] = sub["layers"][:k]
        if sub.get("loop"):
            sub["loop"]["stop"] = min(sub["loop"]["stop"], k)
            if sub["loop"]["start"] >= sub["loop"]["stop"]:
                del sub["loop"]
        keep = {n: t for n, t in w.items() if not (n[0] == "l" and n[1].isdigit()) or int(n[1:n.index(".")]) < k}
        if cfg.get("token_side"):
            keep["side.embed"] = w["side.embed"][:, :k * cfg["token_side"]["dim"]]
        sd = d + f"_first{k}"
        SM.write_model(sub, sd, weights=keep)
        eng = _engine(sd, dtype, PAGE[name], 64)
        logits = eng.step([StepEntry("a", toks, list(range(len(toks))))]).cpu()
        _check({("a", p): logits[p] for p in range(len(toks))}, {"a": PS.forward(sub, keep, toks)}, dtype,
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
@pytest.mark.parametrize("name", ["S1", "S3", "S4"])
def test_long_decoding(models, name, dtype):
    """A short prompt, then 150 tokens one by one: the state moves on 150 times, the window passes over decoded
    tokens, blocks close under them, pages fill, begin and go back; decode steps are replayed from graphs after the
    first two."""
    d, cfg, w, *_ = models[name]
    reqs, ref = _requests(cfg, w, (160,), 3)
    cost = max((PS.forward(cfg, w, t, round_to=torch.float32) - ref[r]).abs().max().item() / ref[r].pow(2).mean().sqrt().item()
               for r, t in reqs.items())
    F32_TOL[name] = max(F32_TOL[name], 8.0 * cost)
    eng = _engine(d, dtype, 16, 12)
    got = TT.run_steps(eng, TT.trace_tail_one_by_one(reqs, 150))
    _check(got, ref, dtype, f"{name} {dtype} long decoding", name)
    assert eng.graph_replays > 100


def test_greedy_generation_through_the_scheduler(models):
    """Runtime.generate_batch (scheduler, portions, the sampler's argmax) against the plain model's greedy tokens,
    in 32-bit; prompts of unequal length, more requests than run at once."""
    from infernum_amd import BatchConfig, GenerateOptions, Runtime
    d, cfg, w, *_ = models["S1"]
    prompts = list(TT.make_requests(cfg["vocab"], (5, 31, 2, 18, 9), seed=9).values())
    rt = Runtime.from_pretrained(d, dtype="float32", batch_config=BatchConfig(block_size=16, num_blocks=24,
                                                                              max_batch_size=3, max_prefill_tokens=8,
                                                                              max_tokens_per_step=16, step_token_multiple=1))
    outs = rt.generate_batch(prompts, GenerateOptions(max_new_tokens=12))
    for p, got in zip(prompts, outs):
        toks = list(p)
        for _ in range(12):
            toks.append(int(PS.forward(cfg, w, toks)[-1].argmax()))
        assert list(got) == toks[len(p):], (p, got, toks[len(p):])


@BOTH
def test_trace_run_and_generate_programs(models, tmp_path, dtype):
    """bin/trace_run and bin/generate as a user starts them: the model class comes from config.json; steps on standard
    input, logits in files; generated tokens on standard output."""
    import json
    import os
    import subprocess
    import sys
    import numpy as np
    d, cfg, w, _, _, reqs, ref = models["S3"]
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
    _check(got, ref, dtype, f"trace_run S3 {dtype} mixed", "S3")
    if dtype == "float32":
        prompt = reqs["r4"][:9]
        gen = subprocess.run([sys.executable, os.path.join(root, "bin", "generate"), "-m", d, "--prompt-ids",
                              ",".join(map(str, prompt)), "-n", "6", "--greedy", "--dtype", "float32"],
                             text=True, capture_output=True, timeout=600)
        assert gen.returncode == 0, gen.stderr[-3000:]
        toks = list(prompt)
        for _ in range(6):
            toks.append(int(PS.forward(cfg, w, toks)[-1].argmax()))
        assert " " + " ".join(map(str, toks[9:])) + "\n" in gen.stdout, gen.stdout[-2000:]
