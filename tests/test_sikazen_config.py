"""The Sikazen configuration reader and model spec on the CPU, and pins of the plain implementation."""
import copy
import math

import pytest
import torch

import plain_sikazen as PS
import sikazen_models as SM
from infernum_amd import models  # noqa: F401  (registers the architectures)
from infernum_amd.config.base import ConfigError
from infernum_amd.config.registry import config_from_dict, model_spec_for
from infernum_amd.config.sikazen import SikazenConfig
from infernum_amd.models.model import DecoderModel
from infernum_amd.parts.base import Runtime

CPU = Runtime(torch.device("cpu"), torch.float32)
F64 = torch.float64


@pytest.mark.parametrize("name", list(SM.RAW))
def test_reads_every_key_and_writes_it_back(name):
    raw = SM.RAW[name]
    cfg = config_from_dict(raw)
    assert isinstance(cfg, SikazenConfig)
    want = copy.deepcopy(raw)
    want.setdefault("embedding", {"scale": 1.0})
    assert cfg.to_dict() == want
    assert config_from_dict(cfg.to_dict()) == cfg


@pytest.mark.parametrize("name", list(SM.RAW))
def test_the_spec_wants_the_tensors_of_the_file_and_runs_the_layers_in_the_plain_order(name):
    raw = SM.RAW[name]
    cfg = config_from_dict(raw)
    model = DecoderModel(model_spec_for(cfg), CPU)
    want = {k: tuple(v.shape) for k, v in model.expected_weights().items() if v.write_when_random}
    assert want == PS.tensor_shapes(raw)
    runs = PS.layer_runs(raw)
    assert [e.layer for e in model.spec.schedule] == [i for i, _ in runs]
    # the embedding's rows are added before a run exactly where the schedule's pass begins anew
    start = raw["loop"]["start"] if raw.get("loop") else -1
    assert [e.pass_index > 0 and e.layer == start for e in model.spec.schedule] == [again for _, again in runs]
    assert all(e.cache_of is None for e in model.spec.schedule)


def test_what_every_mixer_keeps():
    model = DecoderModel(model_spec_for(config_from_dict(SM.S1)), CPU)
    needs = model.cache_needs()
    # two passes of (attention with its blocks, latent attention, recurrence)
    assert len(needs) == 8
    att, blocks, lat, rec = needs[:4]
    assert att[0].kind == "window" and att[0].window == 20 and att[1] is None
    assert {p.name: (p.shape, p.every) for p in blocks[0].payload} == {"pk": ((2, 16), 6), "pv": ((2, 32), 6)}
    assert blocks[0].kind == "full"
    assert blocks[0].payload[0].pool_shape(10, 16) == (10, 2, 3, 16) and blocks[0].payload[0].pool_shape(10, 4) == (10, 2, 1, 16)
    assert lat[0].kind == "full" and lat[0].num_kv_heads == 1 and lat[0].head_dim == 16 + 32
    assert rec[0] is None and rec[1].shape[0] >= 3 * 16 * 32
    # a window shorter than its blocks keeps the open block's pages
    model = DecoderModel(model_spec_for(config_from_dict(SM.S2)), CPU)
    assert model.cache_needs()[0][0].window == 9


@pytest.mark.parametrize("change, message", [
    (lambda c: c["layers"][0].__setitem__("type", "conv"), "type"),
    (lambda c: c["layers"][0]["mixer"].__setitem__("kv_heads", 4), "multiple"),
    (lambda c: c["layers"][0]["mixer"]["rot"].__setitem__("dims", 7), "even"),
    (lambda c: c["layers"][0]["mixer"]["mask"].pop("size"), "size"),
    (lambda c: c["loop"].__setitem__("stop", 9), "loop"),
    (lambda c: c.pop("norm"), "norm"),
    (lambda c: c["layers"][1]["mixer"].pop("kv_rank"), "kv_rank"),
])
def test_a_wrong_configuration_is_refused(change, message):
    raw = copy.deepcopy(SM.S1)
    change(raw)
    with pytest.raises(ConfigError, match=message):
        config_from_dict(raw)


# ------------------------------------------------------------------------------------- pins of the plain model
def test_plain_pooled_window_by_brute_force():
    torch.manual_seed(0)
    T, d, size, pool = 23, 4, 5, 3
    q, k, v = torch.randn(T, d, dtype=F64), torch.randn(T, d, dtype=F64), torch.randn(T, 2, dtype=F64)
    B = T // pool
    kp, vp = k[:B * pool].view(B, pool, d).mean(1), v[:B * pool].view(B, pool, 2).mean(1)
    wk, wb = PS.pooled_window_weights(q @ k.T, q @ kp.T, size, pool)
    for i in range(T):
        keys = [j for j in range(T) if 0 <= i - j < size]
        blocks = [b for b in range(B) if b * pool + pool - 1 <= i - size]
        # nothing is seen twice, and what lies between the blocks and the window is not seen at all
        assert all(b * pool + pool - 1 < min(keys) for b in blocks)
        e = torch.tensor([float(q[i] @ k[j]) for j in keys] + [float(q[i] @ kp[b]) for b in blocks], dtype=F64).exp()
        e = e / e.sum()
        assert torch.allclose(wk[i, keys], e[:len(keys)]) and torch.allclose(wb[i, blocks], e[len(keys):])
        assert float(wk[i].sum() + wb[i].sum()) == pytest.approx(1.0)
        assert wk[i, [j for j in range(T) if j not in keys]].abs().sum() == 0
    # position 7 (window 3..7) sees block 0 (positions 0..2) and not yet block 1 (3..5); position 10 sees block 1
    assert wb[7, 0] > 0 and wb[7, 1] == 0 and wb[10, 1] > 0 and wb[4, 0] == 0


def test_plain_sink_takes_its_share_and_nothing_else():
    torch.manual_seed(1)
    s = torch.randn(6, 6, dtype=F64)
    w = PS.sink_softmax(s, 0.7)
    for i in range(6):
        e = s[i, :i + 1].exp()
        assert torch.allclose(w[i, :i + 1], e / (e.sum() + math.exp(0.7)))
        assert w[i, i + 1:].abs().sum() == 0
    assert torch.allclose(PS.sink_softmax(s, -1e9), torch.softmax(s.masked_fill(torch.triu(torch.ones(6, 6, dtype=torch.bool), 1), -math.inf), 1))


def test_plain_rotation_layouts_and_scaling():
    x = torch.arange(8, dtype=F64).view(1, 1, 8) + 1
    ang = PS.rotation_angles(torch.tensor([3]), 4, 100.0, 2.0)
    assert torch.allclose(ang, torch.tensor([[3 * 1.0 / 2.0, 3 * 100.0 ** -0.5 / 2.0]], dtype=F64))
    half, pairs = PS.rotate(x, ang, 4, "half"), PS.rotate(x, ang, 4, "pairs")
    c, s = torch.cos(ang[0]), torch.sin(ang[0])
    assert torch.allclose(half[0, 0, :4], torch.stack([1 * c[0] - 3 * s[0], 2 * c[1] - 4 * s[1], 3 * c[0] + 1 * s[0], 4 * c[1] + 2 * s[1]]))
    assert torch.allclose(pairs[0, 0, :4], torch.stack([1 * c[0] - 2 * s[0], 2 * c[0] + 1 * s[0], 3 * c[1] - 4 * s[1], 4 * c[1] + 3 * s[1]]))
    assert torch.equal(half[0, 0, 4:], x[0, 0, 4:]) and torch.equal(pairs[0, 0, 4:], x[0, 0, 4:])
    # the unit norm of a head does not care whether it comes before or after the rotation
    assert torch.allclose(PS.unit_rms(half, 0.0), PS.rotate(PS.unit_rms(x, 0.0), ang, 4, "half"))


def test_plain_recurrence_is_a_weighted_sum_of_the_values():
    torch.manual_seed(2)
    T, d, dv = 9, 3, 2
    q, v = torch.randn(T, d, dtype=F64), torch.randn(T, dv, dtype=F64)
    f = torch.rand(T, d, dtype=F64)
    o, S = PS.hgrn2_recurrence(q, f, v)
    for t in range(T):
        want = torch.zeros(dv, dtype=F64)
        for s in range(t + 1):
            keep = torch.ones(d, dtype=F64)
            for r in range(s + 1, t + 1):
                keep = keep * f[r]
            want += (q[t] * keep * (1 - f[s])).sum() * v[s]
        assert torch.allclose(o[t], want)
    # carried on from a state as if uncut
    o1, S1 = PS.hgrn2_recurrence(q[:4], f[:4], v[:4])
    o2, S2 = PS.hgrn2_recurrence(q[4:], f[4:], v[4:], S1)
    assert torch.allclose(torch.cat([o1, o2]), o) and torch.allclose(S2, S)
    # a gate of one keeps everything and takes nothing in
    o3, S3 = PS.hgrn2_recurrence(q, torch.ones(T, d, dtype=F64), v, S)
    assert torch.allclose(S3, S)


def test_plain_latent_scores_are_those_of_the_absorbed_form():
    """(Uk c) . q = c . (Uk^T q): what lets the cache hold the latent alone."""
    torch.manual_seed(3)
    Uk, c, q = torch.randn(5, 7, dtype=F64), torch.randn(7, dtype=F64), torch.randn(5, dtype=F64)
    assert float((Uk @ c) @ q) == pytest.approx(float(c @ (Uk.T @ q)))


def test_plain_model_adds_the_embedding_before_later_passes_only():
    raw = SM.S3
    w = PS.random_weights(raw, 3)
    toks = [5, 9, 200, 31, 7]
    streams = []
    PS.forward(raw, w, toks, streams=streams)
    assert len(streams) == 1 + 3 * 2 + 1
    # the prefix property: a token's logits do not depend on later tokens
    a, b = PS.forward(raw, w, toks), PS.forward(raw, w, toks[:3])
    assert torch.allclose(a[:3], b)
    # without the loop's re-entry the streams differ from the second pass on
    flat = copy.deepcopy(raw)
    flat["loop"]["times"] = 1
    s1 = []
    PS.forward(flat, w, toks, streams=s1)
    assert len(s1) == 4 and torch.equal(s1[2], streams[2]) and not torch.allclose(s1[3], streams[3])
