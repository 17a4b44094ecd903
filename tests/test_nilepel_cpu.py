"""Nilepel without a GPU: configuration, registry, declared tensors, cache needs and the order of the runs, the
rotations' tables, and the plain model's own mechanisms (the oracle of the GPU tests) against properties that do not
depend on it."""
import copy
import math

import pytest
import torch

import plain_nilepel as P
from nilepel_cases import CONFIGS, model_folder, plain_model, tokens_for
from synaptix_amd.config import NilepelConfig, ConfigError, load_config
from synaptix_amd.models import LayerRun
from synaptix_amd.parts import KvNeed, RotaryByWavelength, RotaryInterleaved

F64 = torch.float64


def test_configuration_to_a_dict_and_back():
    for name, d in CONFIGS.items():
        cfg = NilepelConfig.from_dict(copy.deepcopy(d))
        assert NilepelConfig.from_dict(cfg.to_dict()) == cfg, name
    cfg = NilepelConfig.from_dict(copy.deepcopy(CONFIGS["Q"]))
    assert cfg.embedding_scale == 1.0 and cfg.layers[0].mlp.groups == 1 and cfg.layers[0].mlp.route_scale == 1.0
    assert cfg.layers[0].mlp.shared_ff is None and cfg.layers[2].mixer.rot.scaling is None and cfg.layers[3].mlp is None
    assert cfg.layers[3].mixer.window is None and cfg.layers[4].mixer.chunk is None and cfg.layers[2].mixer.kv_from is None


@pytest.mark.parametrize("path,value,word", [
    (("layers", 0, "type"), "conv", "layer type"),
    (("layers", 0, "mixer", "kv_heads"), 3, "kv heads"),
    (("layers", 0, "mixer", "rot", "dims"), 7, "dims"),
    (("layers", 0, "mixer", "rot", "scaling", "high"), 0.5, "low < high"),
    (("layers", 1, "mixer", "rot", "dims"), 10, "dims"),
    (("layers", 3, "mixer", "kv_from"), 3, "earlier layer"),
    (("layers", 3, "mixer", "kv_from"), 1, "another kind"),
    (("layers", 3, "mixer", "heads"), 2, "other head sizes"),
    (("layers", 1, "mlp", "router", "top"), 4, "top"),
    (("layers", 1, "mlp", "router", "groups", "count"), 4, "groups"),
    (("layers", 0, "mlp", "limit"), -1.0, "limit"),
    (("layers", 0, "mlp", "kind"), "glu", "kind"),
    (("norm", "eps"), 0.0, "eps"),
])
def test_errors_name_the_key(path, value, word):
    d = copy.deepcopy(CONFIGS["P"])
    at = d
    for k in path[:-1]:
        at = at[k]
    at[path[-1]] = value
    with pytest.raises(ConfigError) as e:
        NilepelConfig.from_dict(d)
    assert word in str(e.value)


def test_registry_builds_from_a_folder_and_declares_tensors_needs_and_runs():
    arch, cfg = load_config(model_folder("P"))
    assert arch.name == "Nilepel"
    model = arch.build(cfg)
    specs = model.tensor_specs()
    for n in ("embed", "head", "final.norm", "l0.mix.q.b", "l0.mix.k.norm", "l0.mix.sink", "l0.mix.g", "l0.mlp.gate",
              "l1.mix.dkv.norm", "l1.mix.uk", "l1.mlp.e5.gate", "l1.mlp.router", "l1.mlp.shared.sg", "l2.mix.sink",
              "l3.mix.q.norm", "l3.mix.g"):
        assert n in specs, n
    for n in ("l3.mix.k", "l3.mix.v", "l3.mix.k.b", "l3.mix.v.b", "l3.mix.k.norm",      # keys and values are layer 0's
              "l2.norm2", "l2.mix.q.b", "l2.mix.g", "l1.mix.sink", "l1.mlp.correction", "l1.mlp.e6.gate"):
        assert n not in specs, n
    assert specs["l0.mix.g"].shape == (4, 64) and specs["l1.mlp.shared.sg"].shape == (1, 64)
    assert specs["l1.mix.dkv"].shape == (32 + 8, 64) and specs["l2.mix.q"].shape == (6 * 16, 64)
    # layer 3 reads layer 0's cache through a longer window: the cache keeps that one, for both
    assert model.schedule == [LayerRun(0, 0), LayerRun(1, 1), LayerRun(2, 2), LayerRun(3, 0), LayerRun(4, 3)]
    needs = model.cache_needs()
    assert needs[0] == KvNeed(2, 16, 37, v_dim=24)
    assert needs[1] == KvNeed(1, 32 + 8, 33, v_dim=32)
    assert needs[2] == KvNeed(3, 16, 24, v_dim=8)                # a run of 24 positions never reaches further back
    assert needs[3] == KvNeed(1, 16 + 4, 5, v_dim=16)
    assert model.blocks[0].mixer.window == 20 and model.blocks[3].mixer.window == 37 and model.blocks[3].mixer.shared_kv


def test_a_chain_of_readers_and_a_reader_without_a_mask():
    arch, cfg = load_config(model_folder("R"))
    model = arch.build(cfg)
    assert [r.cache for r in model.schedule] == [0, 1, 0, 2, 0]
    assert model.cache_needs()[0] == KvNeed(2, 64, None, v_dim=32)      # one reader sees every key: everything stays
    assert cfg.kv_source(4) == 0 and cfg.kv_source(2) == 0 and cfg.kv_source(1) == 1


@pytest.mark.parametrize("scaling", [None, (4.0, 1.0, 4.0, 64), (8.0, 1.0, 2.0, 128), (3.0, 2.0, 5.0, 1000)])
@pytest.mark.parametrize("base,dims", [(10000.0, 8), (300.0, 32), (1e6, 64)])
def test_tables_of_the_stretched_rotation(base, dims, scaling):
    kw = {} if scaling is None else dict(zip(("factor", "low", "high", "original"), scaling))
    pos = RotaryByWavelength(base, dims, 200, **kw)
    f = P.rates(base, dims)
    want = f if scaling is None else P.stretched_rates(f, *scaling)
    assert torch.allclose(torch.from_numpy(pos.rates()), want, rtol=1e-13, atol=0)
    cos, sin = pos.tables("cpu")
    assert cos.shape == (200, dims // 2)
    ang = torch.arange(200, dtype=F64)[:, None] * want[None, :]
    assert float((cos.double() - torch.cos(ang)).abs().max()) < 1e-7 and float((sin.double() - torch.sin(ang)).abs().max()) < 1e-7
    if scaling is not None:
        factor, low, high, original = scaling
        wave = 2 * math.pi / f
        kinds = {"kept": wave < original / high, "stretched": wave > original / low}
        assert torch.equal(want[kinds["kept"]], f[kinds["kept"]])
        assert torch.allclose(want[kinds["stretched"]], f[kinds["stretched"]] / factor)
        between = ~kinds["kept"] & ~kinds["stretched"]
        assert bool(((want[between] < f[between]) & (want[between] > f[between] / factor)).all())


def test_all_three_kinds_of_waves_occur_in_the_test_configurations():
    f = P.rates(1e6, 32)
    wave = 2 * math.pi / f
    assert bool((wave < 128 / 2.0).any()) and bool((wave > 128 / 1.0).any()) and bool(((wave >= 64) & (wave <= 128)).any())


def test_pairs_and_halves_share_their_tables():
    a, b = RotaryInterleaved(500.0, 12, 50), RotaryByWavelength(500.0, 12, 50, pairing="pairs")
    assert a.pairing == "pairs" and b.pairing == "pairs" and RotaryByWavelength(500.0, 12, 50).pairing == "halves"
    assert torch.equal(a.tables("cpu")[0], b.tables("cpu")[0]) and torch.equal(a.tables("cpu")[1], b.tables("cpu")[1])


# ----------------------------------------------------------------------------- the plain model's own mechanisms
@pytest.mark.parametrize("layout", ["pairs", "halves"])
def test_rotation_keeps_lengths_and_scores_depend_on_the_distance(layout):
    g = torch.Generator().manual_seed(1)
    f = P.rates(100.0, 6)
    x = torch.randn(9, 2, 10, generator=g, dtype=F64)
    y = P.rotate(x, f, layout)
    assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1)) and torch.equal(y[..., 6:], x[..., 6:]) and torch.allclose(y[0], x[0])
    q, k = torch.randn(1, 1, 10, generator=g, dtype=F64), torch.randn(1, 1, 10, generator=g, dtype=F64)
    s = [float((P.rotate(q, f, layout, first=a + 3)[0, 0] * P.rotate(k, f, layout, first=a)[0, 0]).sum()) for a in (0, 5, 40)]
    assert abs(s[0] - s[1]) < 1e-12 and abs(s[0] - s[2]) < 1e-12
    # the two layouts pair other values: on the same input they differ
    assert not torch.allclose(P.rotate(x, f, "pairs"), P.rotate(x, f, "halves"))


def test_masks():
    w = P.window_mask(10, 3)
    assert w[5].tolist() == [False] * 3 + [True] * 3 + [False] * 4 and w[0].tolist() == [True] + [False] * 9
    assert P.window_mask(4, None).tolist() == torch.tril(torch.ones(4, 4)).bool().tolist()
    c = P.chunk_mask(10, 4)
    assert c[5].tolist() == [False] * 4 + [True] * 2 + [False] * 4        # position 5 lies in the run 4..7
    assert c[4].tolist() == [False] * 4 + [True] + [False] * 5 and c[3].tolist() == [True] * 4 + [False] * 6
    assert torch.equal(P.chunk_mask(6, 1), torch.eye(6).bool())


def test_the_sink_takes_weight_and_gives_nothing():
    g = torch.Generator().manual_seed(2)
    q, k, v = (torch.randn(5, 2, 4, generator=g, dtype=F64) for _ in range(3))
    mask = P.window_mask(5, None)
    plain = P.attend(q, k, v, 0.5, mask)
    low = P.attend(q, k, v, 0.5, mask, torch.tensor([-50.0, -50.0], dtype=F64))
    assert torch.allclose(plain, low)
    high = P.attend(q, k, v, 0.5, mask, torch.tensor([0.0, 60.0], dtype=F64))
    assert float(high[:, 1].abs().max()) < 1e-20 and float(high[:, 0].abs().max()) > 1e-3
    # the first token sees itself only: its result is v_0 / (1 + exp(sink - score))
    s0 = 0.5 * float((q[0, 0] * k[0, 0]).sum())
    assert torch.allclose(high[0, 0], v[0, 0] / (1.0 + math.exp(0.0 - s0)))


def test_router_groups_and_weights():
    z = torch.tensor([[0.0, 3.0, 1.0, 2.9, 2.8, -1.0]], dtype=F64)
    s = torch.softmax(z, -1)
    ids, w = P.route(z, 2, 1, 1, 1.0)
    assert ids.tolist() == [[1, 3]] and torch.allclose(w, s[:, [1, 3]])
    ids, w = P.route(z, 2, 3, 1, 2.0)                     # groups {0,1} {2,3} {4,5}: only the first stays
    assert ids.tolist() == [[1, 0]] and torch.allclose(w, 2.0 * s[:, [1, 0]])
    ids, _ = P.route(z, 2, 3, 2, 1.0)                     # the two best groups: {0,1} and {2,3}
    assert ids.tolist() == [[1, 3]]
    ids, _ = P.route(z, 3, 2, 1, 1.0)                     # groups {0,1,2} {3,4,5}: best scores 3.0 and 2.9
    assert sorted(ids.tolist()[0]) == [0, 1, 2]


def test_bounded_feed_forward_clips_both_inputs():
    w = {"gate": torch.tensor([[10.0], [-10.0]], dtype=F64), "up": torch.tensor([[10.0], [-10.0]], dtype=F64),
         "down": torch.eye(2, dtype=F64)}
    y = P.bounded_mlp(torch.ones(1, 1, dtype=F64), w, "", 1.5)
    g0, g1 = 1.5, -10.0
    want = [g0 / (1 + math.exp(-1.702 * g0)) * (1.5 + 1.0), g1 / (1 + math.exp(-1.702 * g1)) * (-1.5 + 1.0)]
    assert torch.allclose(y, torch.tensor([want], dtype=F64))


def test_shared_keys_are_the_owners_keys():
    """The layer that reads another layer's keys gives the same result as that layer would with the reader's queries."""
    m = plain_model("P")
    toks = tokens_for("P", 50, 1)
    c = m.c["layers"]
    h = torch.randn(50, 64, generator=torch.Generator().manual_seed(3), dtype=F64)
    _, kv = P.attention_windowed(h, m.w, "l0.mix.", c[0]["mixer"], 1e-6)
    own, _ = P.attention_windowed(h, m.w, "l3.mix.", c[3]["mixer"], 1e-6, kv)
    w2 = dict(m.w)
    for n in ("k", "k.b", "v", "v.b", "k.norm"):
        w2["l3.mix." + n] = m.w["l0.mix." + n]
    mixer = {k: v for k, v in c[3]["mixer"].items() if k != "kv_from"}
    again, _ = P.attention_windowed(h, w2, "l3.mix.", mixer, 1e-6)
    assert torch.allclose(own, again)
    assert len(m.residuals(toks)) == 5
