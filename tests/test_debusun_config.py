"""Debusun's configuration, its turning into a model description, and the plain implementation's own pins, on the CPU."""
import copy
import math

import pytest
import torch

import plain_debusun as plain
from debusun_models import MODELS
from xinfer_amd.config.model_config import ConfigError
from xinfer_amd.models import config_from_dict, family_of


def test_config_round_trip_and_registry():
    for name, t in MODELS.items():
        fam, cfg = config_from_dict(t["config"])
        assert fam is family_of("Debusun") and cfg.architecture == "Debusun"
        assert fam.config_class.from_dict(cfg.to_dict()) == cfg and cfg.to_dict() == t["config"]
        assert len(cfg.layers) == len(t["config"]["layers"])


def test_a_span_that_runs_again_gets_caches_of_its_own_and_a_start():
    from xinfer_amd.engine.model import EMBEDDING_CACHE, CausalLM
    fam, cfg = config_from_dict(MODELS["A"]["config"])
    spec = fam.spec(cfg)
    assert [(e.layer, e.cache_id) for e in spec.schedule] == [(0, None), (1, None), (2, None), (1, 4), (2, 5), (3, None)]
    starts = [(i, e.before["row"], e.before["add_first"]) for i, e in enumerate(spec.schedule) if e.before is not None]
    assert starts == [(1, 0, False), (3, 1, True)] and spec.schedule[1].before["rows"] == 2
    names = [d.name for d in CausalLM.declare(spec)]
    assert len(names) == len(set(names))
    for want in ("embed", "bigram", "loop.step", "l0.mix.in", "l0.mix.conv.b", "l0.mix.A_log", "l1.mix.q", "l2.mix.dkv.norm",
                 "l2.mix.sink", "l2.mix.g", "l3.mlp.up", "final.norm", "head"):
        assert want in names
    assert not any(n.startswith(("l1.mlp", "l1.norm2")) for n in names)
    model = CausalLM(spec, torch.float32)
    assert sorted(model.kv_needs) == [1, 2, 3, 4, 5] and [g.window for g in model.cache_groups] == [12, 21, 30]
    assert sorted(model.state_needs) == [EMBEDDING_CACHE, 0]
    state, tail = model.state_needs[0]
    assert state.shape == (4, 16, 24) and tail.shape == (2, 4 * 24 + 2 * 2 * 16) and tail.name == "conv_tail"
    assert model.state_needs[EMBEDDING_CACHE].dtype == torch.int32
    assert model.kv_needs[2].pools[0].shape[-1] == 48 and len(model.kv_needs[2].pools) == 1      # the latent and the turned part
    # value heads of their own size: a head at a time; equal sizes: the plain form's kernels
    assert model.blocks[1].mixer.by_head and not model.blocks[3].mixer.general and model.blocks[3].mixer.unit_norm


def test_spans_that_cover_everything_run_once_or_are_absent():
    fam, cfg = config_from_dict(MODELS["B"]["config"])
    spec = fam.spec(cfg)
    assert [(e.layer, e.cache_id) for e in spec.schedule] == [(0, None), (1, None), (2, None), (0, 3), (1, 4), (2, 5), (0, 6), (1, 7), (2, 8)]
    assert [i for i, e in enumerate(spec.schedule) if e.before is not None] == [0, 3, 6]
    assert [e.before["add_first"] for e in spec.schedule if e.before is not None] == [False, True, True]
    fam, cfg = config_from_dict(MODELS["C"]["config"])
    spec = fam.spec(cfg)
    assert all(e.before is None and e.cache_id is None for e in spec.schedule) and len(spec.schedule) == 4
    from xinfer_amd.engine.model import CausalLM
    assert "loop.step" not in [d.name for d in CausalLM.declare(spec)]
    fam, cfg = config_from_dict(MODELS["D"]["config"])
    spec = fam.spec(cfg)
    assert [(e.layer, e.cache_id, e.before is not None) for e in spec.schedule] == [(0, None, False), (1, None, True), (2, None, False)]
    assert spec.schedule[1].before["rows"] == 1 and not spec.schedule[1].before["add_first"]


@pytest.mark.parametrize("change,message", [
    (lambda c: c["layers"][0].update(type="conv"), "unknown layer type"),
    (lambda c: c["layers"][1]["mixer"].update(kv_heads=4), "kv heads"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=7), "even"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=64), "rotated dims"),
    (lambda c: c["layers"][2]["mixer"].update(rot_dim=6), "rot.dims"),
    (lambda c: c["layers"][0]["mixer"].update(groups=3), "groups"),
    (lambda c: c["layers"][0]["mlp"].update(kind="moe"), "mlp kind"),
    (lambda c: c["loop"].update(stop=9), "loop"),
    (lambda c: c["loop"].update(times=0), "loop"),
    (lambda c: c["embedding"]["bigram"].update(buckets=0), "buckets"),
    (lambda c: c.pop("norm"), "norm"),
])
def test_configurations_that_cannot_be_run(change, message):
    raw = copy.deepcopy(MODELS["A"]["config"])
    change(raw)
    with pytest.raises(ConfigError, match=message):
        config_from_dict(raw)


# ---- what fixes each rule of the plain implementation beside its text ------------------------------------------
def test_pair_rows():
    assert plain.bigram_rows([5, 9, 9, 0], 7, 3, 2) == [7, (15 + 18) % 7, (27 + 18) % 7, 27 % 7]


def test_ramp_of_the_frequencies_and_the_tables_of_the_engine():
    rot = dict(dims=16, base=10000.0, scaling=dict(factor=4.0, original=64, fast=8.0, slow=1.0))
    f, m = plain.rotary_frequencies(rot)
    base_f, one = plain.rotary_frequencies(dict(dims=16, base=10000.0))
    ratio = (f / base_f).tolist()
    assert one == 1.0 and abs(m - (0.1 * math.log(4.0) + 1)) < 1e-12
    assert ratio[0] == 1.0 and abs(ratio[-1] - 0.25) < 1e-12 and any(0.26 < r < 0.99 for r in ratio)
    assert all(a >= b for a, b in zip(ratio, ratio[1:]))
    from xinfer_amd.parts.rope import scaled_inv_freq
    inv, mm = scaled_inv_freq(10000.0, 16, dict(kind="ramp", factor=4.0, original=64, fast=8.0, slow=1.0))
    assert abs(mm - m) < 1e-12 and torch.allclose(torch.from_numpy(inv).double(), f, rtol=1e-6)


def test_rotation_turns_neighbours_and_keeps_lengths():
    x = torch.randn(5, 2, 12, dtype=torch.float64)
    rot = dict(dims=8, base=100.0)
    y = plain.rotate(x, rot, torch.arange(5))
    assert torch.equal(y[0], x[0]) and torch.equal(y[..., 8:], x[..., 8:])
    assert torch.allclose((y ** 2).sum(-1), (x ** 2).sum(-1))
    a = 3 * 100.0 ** (-2 / 8)       # position 3, pair 1
    assert torch.allclose(y[3, 0, 2], x[3, 0, 2] * math.cos(a) - x[3, 0, 3] * math.sin(a))
    assert torch.allclose(y[3, 0, 3], x[3, 0, 3] * math.cos(a) + x[3, 0, 2] * math.sin(a))


def test_window_and_sink():
    s = torch.zeros(6, 6, dtype=torch.float64)
    p = plain.window_softmax(s, 3)
    assert torch.allclose(p[5], torch.tensor([0, 0, 0, 1 / 3, 1 / 3, 1 / 3], dtype=torch.float64))
    assert torch.allclose(p[1], torch.tensor([0.5, 0.5, 0, 0, 0, 0], dtype=torch.float64))
    p = plain.window_softmax(s, 3, sink=torch.tensor(math.log(3.0), dtype=torch.float64))
    assert torch.allclose(p[5].sum(), torch.tensor(0.5, dtype=torch.float64)) and torch.allclose(p[0, 0], torch.tensor(0.25, dtype=torch.float64))


def test_the_state_goes_on_where_a_portion_ended_and_the_convolution_sees_no_earlier_sequence():
    g = torch.Generator().manual_seed(1)
    T, H, dv, G, N = 9, 4, 3, 2, 5
    x, B, C = (torch.randn(T, *s, generator=g, dtype=torch.float64) for s in ((H, dv), (G, N), (G, N)))
    dt = torch.rand(T, H, generator=g, dtype=torch.float64)
    a, skip = torch.randn(H, generator=g, dtype=torch.float64), torch.randn(H, generator=g, dtype=torch.float64)
    y, S = plain.state_space(x, B, C, dt, a, skip)
    y1, S1 = plain.state_space(x[:4], B[:4], C[:4], dt[:4], a, skip)
    y2, S2 = plain.state_space(x[4:], B[4:], C[4:], dt[4:], a, skip, state=S1)
    assert torch.allclose(torch.cat([y1, y2]), y) and torch.allclose(S2, S)
    # the first token's result is its own share alone
    assert torch.allclose(y[0, 3], dt[0, 3] * (B[0, 1] @ C[0, 1]) * x[0, 3] + skip[3] * x[0, 3])
    u = torch.randn(6, 2, generator=g, dtype=torch.float64)
    w, b = torch.randn(2, 3, generator=g, dtype=torch.float64), torch.randn(2, generator=g, dtype=torch.float64)
    out = plain.causal_conv(u, w, b)
    assert torch.allclose(out[0], b + w[:, 2] * u[0]) and torch.allclose(out[2], b + w[:, 0] * u[0] + w[:, 1] * u[1] + w[:, 2] * u[2])
