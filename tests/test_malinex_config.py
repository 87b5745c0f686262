"""The Malinex configuration reader and model spec on the CPU, and pins of the plain implementation."""
import copy
import math

import pytest
import torch

import malinex_models as MM
import plain_malinex as PM
from infernum_amd import models  # noqa: F401  (registers the architectures)
from infernum_amd.config.base import ConfigError
from infernum_amd.config.malinex import MalinexConfig
from infernum_amd.config.registry import config_from_dict, model_spec_for
from infernum_amd.models.model import DecoderModel
from infernum_amd.parts.base import Runtime

CPU = Runtime(torch.device("cpu"), torch.float32)


@pytest.mark.parametrize("name", list(MM.RAW))
def test_reads_every_key_and_writes_it_back(name):
    raw = MM.RAW[name]
    cfg = config_from_dict(raw)
    assert isinstance(cfg, MalinexConfig)
    back = cfg.to_dict()
    want = copy.deepcopy(raw)
    want.setdefault("logit_scale", 1.0)
    for entry in want["layers"]:
        if entry["type"] == "attention":
            entry["mixer"].setdefault("kv_heads", entry["mixer"]["heads"])
    assert back == want
    assert config_from_dict(back) == cfg


@pytest.mark.parametrize("name", list(MM.RAW))
def test_the_spec_wants_the_tensors_of_the_file(name):
    raw = MM.RAW[name]
    model = DecoderModel(model_spec_for(config_from_dict(raw)), CPU)
    want = {k: tuple(v.shape) for k, v in model.expected_weights().items()}
    assert want == PM.tensor_shapes(raw)
    # a layer that runs with another's tensors is one more run of that layer, with a cache or state of its own
    assert len(model.spec.schedule) == len(raw["layers"])
    assert all(e.cache_of is None for e in model.spec.schedule)
    owners = [entry.get("weights_of", i) for i, entry in enumerate(raw["layers"])]
    own = sorted(set(owners))
    assert [e.layer for e in model.spec.schedule] == [own.index(o) for o in owners]
    for entry, (cs, ss) in zip(raw["layers"], model.cache_needs()):
        m = entry["mixer"]
        if entry["type"] == "gla":
            assert cs is None and ss.shape[0] >= m["heads"] * m["dim"] * m["vdim"]
        else:
            assert ss is None and cs.kind == "full"
            shapes = {p.name: tuple(p.shape) for p in cs.payload}
            G = m.get("kv_heads", m["heads"])
            assert shapes == {"k": (G, m["dim"]), "v": (G, m["vdim"])}


def test_the_width_of_the_decays_middle_comes_from_the_file_when_the_configuration_is_silent():
    raw = copy.deepcopy(MM.X4)
    for entry in raw["layers"]:
        entry["mixer"].pop("rank")
    model = DecoderModel(model_spec_for(config_from_dict(raw)), CPU)
    shapes = {k: tuple(v.shape) for k, v in model.expected_weights().items()}
    assert shapes["l0.mix.a1"] == (-1, raw["width"]) and shapes["l0.mix.a2"][1] == -1
    from infernum_amd.weights.loader import check_against
    check_against(model.expected_weights(), PM.tensor_shapes(MM.X4), "a file")          # any width fits


def test_what_a_file_does_not_mention_is_not_there():
    cfg = config_from_dict(MM.X2)
    assert cfg.logit_scale == 1.0
    att = cfg.layers[0]
    assert att.mixer.kv_heads == att.mixer.heads and att.mixer.q_temp_coef is None and att.mlp is None
    spec = model_spec_for(cfg)
    assert spec.layers[0].feed_forward is None and spec.layers[0].feed_forward_norm is None
    assert set(spec.layers[0].extra) == {"mixer_post_norm", "mixer_gate"}
    assert spec.layers[1].feed_forward.params["shared_ff"] is None
    names = DecoderModel(spec, CPU).expected_weights()
    assert "l0.norm2" not in names and "l0.rg2" not in names and "l1.mlp.shared.up" not in names


@pytest.mark.parametrize("change,match", [
    (lambda c: c["layers"][1]["mixer"].update(kv_heads=3), "kv_heads"),
    (lambda c: c["layers"][0].update(type="window"), "type"),
    (lambda c: c["layers"][0]["mixer"].update(tau=0.0), "tau"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=7), "experts"),
    (lambda c: c["layers"][2].update(weights_of=3), "weights_of"),
    (lambda c: c["layers"][2].update(weights_of=2), "weights_of"),
    (lambda c: c["layers"][2].update(weights_of=1), "sizes"),
    (lambda c: c["layers"][2].update(mixer=dict(c["layers"][2]["mixer"], dim=8)), "sizes"),
    (lambda c: c["layers"][0]["mlp"].update(kind="gated"), "kind"),
    (lambda c: c.pop("norm"), "norm"),
    (lambda c: c["layers"][1].pop("mixer"), "mixer"),
    (lambda c: c.update(layers=[]), "layers"),
])
def test_refuses_what_does_not_fit(change, match):
    raw = copy.deepcopy(MM.X1)
    change(raw)
    with pytest.raises(ConfigError, match=match):
        config_from_dict(raw)


def test_random_weights_from_a_configuration():
    """Every tensor can be drawn when the configuration tells the decays' middle; without it a file is needed."""
    spec = model_spec_for(config_from_dict(MM.X3))
    model = DecoderModel(spec, CPU)
    assert all(-1 not in ws.shape for ws in model.expected_weights().values())


# ------------------------------------------------------------------------ pins of the plain implementation
def _mix(cfg, i, seed=3):
    w = {k: v.double() for k, v in PM.random_weights(cfg, seed).items()}
    p = f"l{i}.mix."
    return {k[len(p):]: v for k, v in w.items() if k.startswith(p)}, w


def test_plain_recurrence_by_hand():
    g = torch.Generator().manual_seed(0)
    q, k, la = (torch.randn(5, 3, generator=g).double() for _ in range(3))
    la = -la.abs()
    v = torch.randn(5, 2, generator=g).double()
    o, S = PM.gla_recurrence(q, k, v, la)
    for t in range(5):
        want = torch.zeros(2, dtype=torch.float64)
        for j in range(t + 1):
            decay = torch.exp(la[j + 1:t + 1].sum(dim=0))            # key j has met the decays after its own token
            want += (q[t] * decay * k[j]).sum() * v[j]
        assert torch.allclose(o[t], want, atol=1e-12)
    o2, _ = PM.gla_recurrence(q[3:], k[3:], v[3:], la[3:], state=PM.gla_recurrence(q[:3], k[:3], v[:3], la[:3])[1])
    assert torch.allclose(o2, o[3:], atol=1e-12)


def test_plain_decay_is_a_root_of_a_sigmoid():
    a = torch.randn(4, 6, dtype=torch.float64)
    wa1, wa2, b = torch.randn(2, 6, dtype=torch.float64), torch.randn(5, 2, dtype=torch.float64), torch.randn(5, dtype=torch.float64)
    la = PM.gla_decays(a, wa1, wa2, b, 4.0)
    assert torch.allclose(torch.exp(la), torch.sigmoid(a @ wa1.T @ wa2.T + b) ** 0.25, atol=1e-12)
    assert (la <= 0).all()


def test_plain_attention_weights_are_causal_unnormalised_and_fall_with_distance():
    g = torch.Generator().manual_seed(1)
    q, k = torch.randn(6, 4, generator=g).double(), torch.randn(6, 4, generator=g).double()
    w = PM.sigmoid_attention_weights(q, k, 0.5, 0.7, 0.3, -1.0)
    assert torch.equal(w.triu(1), torch.zeros_like(w))
    assert math.isclose(float(w[4, 1]), 1 / (1 + math.exp(-(0.5 * float(q[4] @ k[1]) - 0.7 * math.log1p(0.3 * 3) - 1.0))), rel_tol=1e-12)
    assert not torch.allclose(w.sum(dim=1), torch.ones(6, dtype=torch.float64))
    same = PM.sigmoid_attention_weights(torch.ones(9, 4).double(), torch.ones(9, 4).double(), 0.1, 0.5, 1.0, 0.0)
    assert (same[8, :8] < same[8, 1:9]).all()                          # nearer keys weigh more
    # queries that start later: the same rows
    assert torch.allclose(PM.sigmoid_attention_weights(q[3:], k, 0.5, 0.7, 0.3, -1.0, offset=3), w[3:], atol=1e-15)


def test_plain_query_factor_steps():
    f = PM.query_temperature(torch.arange(40), 0.5, 16)
    assert float(f[14]) == 1.0 and math.isclose(float(f[15]), 1 + 0.5 * math.log(2.0)) and float(f[30]) == float(f[15])
    assert math.isclose(float(f[31]), 1 + 0.5 * math.log(3.0))


def test_plain_router_corrects_the_choice_only():
    f, wr = torch.eye(3, dtype=torch.float64), torch.tensor([[2.0, 0, 0], [1.0, 0, 0], [0.0, 0, 0]], dtype=torch.float64)
    chosen, wts = PM.router(f[:1], wr, torch.zeros(3, dtype=torch.float64), 2)
    assert sorted(chosen[0].tolist()) == [0, 1]
    s = torch.softmax(torch.tensor([2.0, 1.0, 0.0], dtype=torch.float64), 0)
    chosen, wts = PM.router(f[:1], wr, torch.tensor([0.0, -1.0, 0.0], dtype=torch.float64), 2)
    assert sorted(chosen[0].tolist()) == [0, 2]
    got = dict(zip(chosen[0].tolist(), wts[0].tolist()))
    assert math.isclose(got[0], float(s[0] / (s[0] + s[2]))) and math.isclose(got[2], float(s[2] / (s[0] + s[2])))


def test_plain_model_is_causal_and_shares_tensors_between_runs():
    cfg = MM.X1
    w = PM.random_weights(cfg, 2)
    assert not any(n.startswith(("l2.", "l3.")) for n in w)
    toks = list(range(3, 40))
    full = PM.forward(cfg, w, toks)
    assert torch.allclose(full[:20], PM.forward(cfg, w, toks[:20]), atol=1e-10)
    streams = []
    PM.forward(cfg, w, toks, streams=streams)
    assert len(streams) == 4
    unscaled = PM.forward(dict(cfg, logit_scale=1.0), w, toks)
    assert torch.allclose(full, unscaled * cfg["logit_scale"], atol=1e-12)
