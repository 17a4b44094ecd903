"""Repolix without a GPU: configuration, registry, declared tensors and cache needs, the rotation's tables, and the
plain model's own mechanisms (the oracle of the GPU tests) against properties that do not depend on it."""
import copy
import math

import pytest
import torch

import plain_repolix as P
from repolix_cases import CONFIGS, model_folder, plain_model, tokens_for
from synaptix_amd.config import RepolixConfig, ConfigError, load_config
from synaptix_amd.parts import KvNeed, StateNeed, RotaryScaledHalfSplit

F64 = torch.float64


def test_configuration_to_a_dict_and_back():
    for name, d in CONFIGS.items():
        cfg = RepolixConfig.from_dict(copy.deepcopy(d))
        again = RepolixConfig.from_dict(cfg.to_dict())
        assert again == cfg, name
    cfg = RepolixConfig.from_dict(copy.deepcopy(CONFIGS["Q"]))
    assert cfg.embedding_scale == 1.0 and cfg.layers[0].mlp.identity == 0 and cfg.layers[0].mlp.groups == 1
    assert cfg.layers[1].mixer.rot_scaling is None and cfg.layers[2].mlp is None


@pytest.mark.parametrize("path,value,word", [
    (("layers", 0, "type"), "conv", "layer type"),
    (("layers", 1, "mixer", "groups"), 3, "groups"),
    (("layers", 0, "mixer", "rot", "dims"), 7, "dims"),
    (("layers", 0, "mlp", "router", "top"), 40, "top"),
    (("layers", 0, "mlp", "router", "groups", "count"), 3, "groups"),
    (("layers", 0, "mlp", "expert", "limit"), -1.0, "limit"),
    (("layers", 2, "mixer", "kv_heads"), 3, "kv heads"),
    (("norm", "eps"), 0.0, "eps"),
])
def test_errors_name_the_key(path, value, word):
    d = copy.deepcopy(CONFIGS["P"])
    at = d
    for k in path[:-1]:
        at = at[k]
    at[path[-1]] = value
    with pytest.raises(ConfigError) as e:
        RepolixConfig.from_dict(d)
    assert word in str(e.value)


def test_registry_builds_from_a_folder_and_declares_tensors_and_needs():
    arch, cfg = load_config(model_folder("P"))
    assert arch.name == "Repolix"
    model = arch.build(cfg)
    specs = model.tensor_specs()
    for n in ("embed", "head", "final.norm", "l0.ls1", "l0.ls2", "l0.mix.q.conv", "l0.mix.lq1", "l0.mlp.e5.gate",
              "l0.mlp.correction", "l0.mlp.shared.down", "l1.mix.conv.b", "l1.mix.A_log", "l2.mix.a2", "l2.mix.g1"):
        assert n in specs, n
    assert "l1.ls2" not in specs and "l1.norm2" not in specs            # a layer without a feed-forward
    assert "l0.mlp.e6.gate" not in specs                                # identity experts have no tensors
    assert specs["l0.mlp.router"].shape == (8, 64)
    needs = model.cache_needs()
    m = cfg.layers[0].mixer
    assert needs[0] == (StateNeed((2, (2 * 4 + 2 * 2) * 16 + 2 * 24)), KvNeed(4, 16, 20, v_dim=24, v_heads=2))
    assert needs[1] == (StateNeed((3, 4 * 16 + 2 * 2 * 24)), StateNeed((4, 24, 16)))
    assert needs[2] == (StateNeed((2, 2 * 2 * 16 + 4 * 24)), StateNeed((4, 16, 24)))
    assert m.window == 20


def test_sizes_that_only_stored_weights_decide():
    """The narrow middles of the delta rule's decays and gate are in no key: the specs leave them open, a file's shapes
    fill them in, and random weights need them named."""
    from synaptix_amd.weights.source import RandomSource
    d = copy.deepcopy(CONFIGS["P"])
    del d["middle_rank"]
    arch, _ = load_config(model_folder("P"))
    model = arch.build(RepolixConfig.from_dict(d))
    spec = model.tensor_specs()["l2.mix.a1"]
    assert spec.shape == (None, 64)
    with pytest.raises(ValueError):
        RandomSource(model.tensor_specs(), 0).tensor("l2.mix.a1")


def test_rotation_tables():
    plain = RotaryScaledHalfSplit(10000.0, 16, 50)
    cos, sin = plain.host_tables()
    assert cos.shape == (50, 8) and abs(float(cos[0].min()) - 1.0) < 1e-7 and float(abs(sin[0]).max()) == 0.0
    rot = {"base": 10000.0, "dims": 16, "scaling": {"factor": 4.0, "original": 64, "fast": 16.0, "slow": 2.0}}
    f, m = P.scaled_frequencies(rot)
    scaled = RotaryScaledHalfSplit(10000.0, 16, 50, factor=4.0, original=64, fast=16.0, slow=2.0)
    rates, mult = scaled.rates()
    assert torch.allclose(torch.from_numpy(rates), f, rtol=1e-12) and abs(mult - m) < 1e-12
    assert abs(m - (0.1 * math.log(4.0) + 1.0)) < 1e-12
    assert float(f[0]) == 1.0 and abs(float(f[-1]) - 10000.0 ** (-14 / 16) / 4.0) < 1e-12     # fast waves kept, slow ones stretched
    cos, sin = scaled.host_tables()
    want = torch.arange(50, dtype=F64)[:, None] * f
    assert float((torch.from_numpy(cos).double() - torch.cos(want) * m).abs().max()) < 1e-5


def test_plain_short_conv_and_rotation():
    g = torch.Generator().manual_seed(1)
    u, w = torch.randn(9, 5, generator=g, dtype=F64), torch.randn(5, 3, generator=g, dtype=F64)
    y = P.short_conv(u, w)
    assert torch.allclose(y[0], w[:, 2] * u[0]) and torch.allclose(y[4], w[:, 0] * u[2] + w[:, 1] * u[3] + w[:, 2] * u[4])
    assert torch.allclose(P.short_conv(u, torch.ones(5, 1, dtype=F64)), u)
    rot = {"base": 100.0, "dims": 4}
    x = torch.randn(7, 2, 6, generator=g, dtype=F64)
    y = P.turn_halves(x, torch.arange(7), rot)
    assert torch.allclose(y[0], x[0]) and torch.allclose(y[..., 4:], x[..., 4:])
    assert torch.allclose(y[..., :4].pow(2).sum(-1), x[..., :4].pow(2).sum(-1))
    # scores depend on the distance only
    q, k = torch.randn(1, 6, generator=g, dtype=F64), torch.randn(1, 6, generator=g, dtype=F64)
    s = [float(P.turn_halves(q, torch.tensor([a + 3]), rot)[0] @ P.turn_halves(k, torch.tensor([a]), rot)[0]) for a in (0, 5, 40)]
    assert abs(s[0] - s[1]) < 1e-12 and abs(s[0] - s[2]) < 1e-12


def test_plain_cells_in_two_pieces():
    """The recurrences carried across a cut equal the whole sequence's."""
    g = torch.Generator().manual_seed(2)
    T, H, Pv, G, N = 12, 4, 3, 2, 5
    r = lambda *s: torch.randn(*s, generator=g, dtype=F64)
    x, B, C, dt = r(T, H, Pv), r(T, G, N), r(T, G, N), r(T, H)
    bias, a_log, d = r(H), r(H) - 1.0, r(H)
    whole = P.state_space_cell(x, B, C, dt, bias, a_log, d)
    S = torch.zeros(H, N, Pv, dtype=F64)
    parts = [P.state_space_cell(x[a:b], B[a:b], C[a:b], dt[a:b], bias, a_log, d, S) for a, b in ((0, 5), (5, 12))]
    assert torch.allclose(torch.cat(parts), whole)
    K, D, E = 2, 6, 3
    q, k, v, beta, a = r(T, K, D), r(T, K, D), r(T, H, E), r(T, H), r(T, H, D)
    whole = P.delta_cell(q, k, v, beta, a, r(H, D) * 0, a_log)
    S = torch.zeros(H, D, E, dtype=F64)
    parts = [P.delta_cell(q[a0:b0], k[a0:b0], v[a0:b0], beta[a0:b0], a[a0:b0], torch.zeros(H, D, dtype=F64), a_log, S)
             for a0, b0 in ((0, 7), (7, 12))]
    assert torch.allclose(torch.cat(parts), whole)
    # with a step of one and no decay the delta rule stores v under k exactly: reading with k gives v back
    one = torch.full((1, 1), 50.0, dtype=F64)
    kk, vv = r(1, 1, D), r(1, 1, E)
    o = P.delta_cell(kk, kk, vv, one, torch.full((1, 1, D), -80.0, dtype=F64), torch.zeros(1, D, dtype=F64), torch.zeros(1, dtype=F64))
    assert torch.allclose(o[0, 0] * D ** 0.5, vv[0, 0], atol=1e-5)


def test_plain_router():
    w = {"r.router": torch.eye(8, dtype=F64)[:, :6] * 0 + torch.randn(8, 6, generator=torch.Generator().manual_seed(3), dtype=F64),
         "r.correction": torch.zeros(8, dtype=F64)}
    h = torch.randn(20, 6, generator=torch.Generator().manual_seed(4), dtype=F64)
    chosen, weights = P.route(h, w, "r.", {"experts": 6, "identity": 2, "top": 3, "groups": {"count": 4, "keep": 2}})
    s = torch.softmax(h @ w["r.router"].T, -1)
    for t in range(20):
        groups = {int(e) // 2 for e in chosen[t]}
        assert len(groups) <= 2
        best = s[t].view(4, 2).max(-1).values
        assert groups <= set(torch.topk(best, 2).indices.tolist())
        assert torch.allclose(weights[t], s[t][chosen[t]]) and float(weights[t].sum()) < 1.0
    # a correction moves the choice and leaves the weights alone
    w["r.correction"] = torch.tensor([0, 0, 0, 0, 0, 0, 5.0, 5.0], dtype=F64)
    chosen2, weights2 = P.route(h, w, "r.", {"experts": 6, "identity": 2, "top": 2, "groups": {"count": 4, "keep": 1}})
    assert all(set(c.tolist()) == {6, 7} for c in chosen2)
    assert torch.allclose(weights2, torch.gather(s, 1, chosen2))


def test_plain_experts_and_the_whole_model_runs():
    h = torch.tensor([[10.0, -10.0]], dtype=F64)
    eye = torch.eye(2, dtype=F64)
    y = P.clamped_expert(h, eye, eye, eye, 1.25)
    g = torch.tensor([1.25, -10.0], dtype=F64)
    u = torch.tensor([1.25, -1.25], dtype=F64)
    assert torch.allclose(y[0], g * torch.sigmoid(1.702 * g) * (u + 1.0))
    toks = tokens_for("P", 30, 1)
    res, lg = plain_model("P").residuals(toks)
    assert res.shape == (4, 30, 64) and lg.shape == (30, 300) and torch.isfinite(lg).all()
    # causal: a later token changes no earlier logit
    other = toks[:20] + tokens_for("P", 10, 2)
    assert torch.allclose(plain_model("P").logits(other)[:20], lg[:20])
