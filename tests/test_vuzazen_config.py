"""Vuzazen's configuration, its turning into a model description, and the plain implementation's own pins, on the CPU."""
import copy
import math

import pytest
import torch

import plain_vuzazen as plain
from vuzazen_models import MODELS
from xinfer_amd.config.model_config import ConfigError
from xinfer_amd.models import config_from_dict, family_of


def test_config_round_trip_and_registry():
    for name, t in MODELS.items():
        fam, cfg = config_from_dict(t["config"])
        assert fam is family_of("Vuzazen") and cfg.architecture == "Vuzazen"
        assert fam.config_class.from_dict(cfg.to_dict()) == cfg and cfg.to_dict() == t["config"]
        assert len(cfg.layers) == len(t["config"]["layers"])


def test_what_the_layers_keep_and_what_their_tensors_are_called():
    from xinfer_amd.engine.model import EMBEDDING_CACHE, CausalLM
    fam, cfg = config_from_dict(MODELS["A"]["config"])
    spec = fam.spec(cfg)
    assert [(e.layer, e.cache_id, e.before) for e in spec.schedule] == [(i, None, None) for i in range(4)]
    names = {d.name: tuple(d.shape) for d in CausalLM.declare(spec)}
    for want, shape in (("embed", (311, 96)), ("bigram", (98, 96)), ("l0.mix.i", (3, 96)), ("l0.mix.f.b", (3,)), ("l0.mix.norm", (72,)),
                        ("l0.mlp.router", (4, 96)), ("l0.mlp.e3.down", (96, 40)), ("l1.mix.q.conv", (96, 3)), ("l1.mix.v.conv", (48, 3)),
                        ("l1.mix.q.norm", (96,)), ("l1.mix.talk", (6, 6)), ("l1.mix.g", (6, 96)), ("l2.mix.dq", (24, 96)),
                        ("l2.mix.dq.norm", (24,)), ("l2.mix.uq", (96, 24)), ("l2.mix.dkv", (48, 96)), ("l2.mix.g", (4, 96)),
                        ("l3.mix.talk", (4, 4)), ("final.norm", (96,))):
        assert names.get(want) == shape, want
    assert not any(n.startswith(("l2.mlp", "l2.norm2", "l3.mix.q.conv", "head", "l2.mix.q")) and n != "l2.mix.q" for n in names)
    assert "l2.mix.q" not in names and "l2.mix.sink" not in names
    model = CausalLM(spec, torch.float32)
    assert model.head.tied and sorted(model.kv_needs) == [1, 2, 3] and [g.window for g in model.cache_groups] == [0]
    assert sorted(model.state_needs) == [EMBEDDING_CACHE, 0, 1]
    state, top = model.state_needs[0]
    assert state.shape == (3, 16, 25) and top.shape == (3,) and top.name == "max"
    assert model.state_needs[1].shape == (2, 6 * 16 + 2 * 16 + 2 * 24) and model.state_needs[1].name == "conv_tail"
    # mixed heads score against a token's whole k row: one key head; the values keep their kv heads
    k, v = model.kv_needs[1].pools
    assert k.shape[0] == 1 and k.shape[-1] == 2 * 16 and v.shape[0] == 2
    assert model.kv_needs[2].pools[0].shape[-1] == 48 and len(model.kv_needs[2].pools) == 1
    assert model.blocks[1].mixer.rows_form and model.blocks[3].mixer.taps == 0 and model.blocks[3].mixer.state_need() is None
    assert model.blocks[2].mixer.head_gate and model.blocks[2].mixer.q_rank == 24 and not model.blocks[2].mixer.has_sinks
    assert model.blocks[0].ffn.sigmoid_scores and model.blocks[0].ffn.weigh_input
    # every norm of the family multiplies by one plus its tensor
    assert model.blocks[0].norm1.weight_offset == 1.0 and model.final_norm.weight_offset == 1.0
    fam, cfg = config_from_dict(MODELS["M"]["config"])
    model = CausalLM(fam.spec(cfg), torch.bfloat16)
    assert not model.kv_needs and sorted(model.state_needs) == [EMBEDDING_CACHE, 0, 1]


def test_a_norm_that_multiplies_by_one_plus_its_tensor():
    from xinfer_amd.config.spec import PartSpec
    from xinfer_amd.parts import norm_class
    from xinfer_amd.weights.store import RandomStore
    spec = PartSpec("rmsnorm", dict(dim=40, eps=1e-5, name="n", weight_offset=1.0))
    cls = norm_class("rmsnorm")
    store = RandomStore(cls.declare(spec, ""), 3, 0.02, 0.1, torch.bfloat16)
    stored = store.get("n", torch.float32, "cpu")
    assert abs(float(stored.mean())) < 0.1 and float(stored.abs().max()) < 0.6
    part = cls(spec, torch.float32)
    part.load(store, "", "cpu")
    assert torch.equal(part.weight, stored + 1.0)


@pytest.mark.parametrize("change,message", [
    (lambda c: c["layers"][0].update(type="conv"), "unknown layer type"),
    (lambda c: c["layers"][1]["mixer"].update(kv_heads=4), "kv heads"),
    (lambda c: c["layers"][2]["mixer"]["rot"].update(dims=7), "even"),
    (lambda c: c["layers"][2]["mixer"].update(rot_dim=6), "rot.dims"),
    (lambda c: c["layers"][2]["mixer"].pop("q_rank"), "q_rank"),
    (lambda c: c["layers"][0]["mixer"].update(gate_cap=0), "gate cap"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=5), "experts cannot be chosen"),
    (lambda c: c["layers"][1]["mlp"].update(kind="sparse"), "mlp kind"),
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


def test_rotation_turns_the_two_halves_and_keeps_lengths():
    x = torch.randn(5, 2, 12, dtype=torch.float64)
    rot = dict(dims=8, base=100.0)
    y = plain.rotate_half(x, rot, torch.arange(5))
    assert torch.equal(y[0], x[0]) and torch.equal(y[..., 8:], x[..., 8:])
    assert torch.allclose((y ** 2).sum(-1), (x ** 2).sum(-1))
    a = 3 * 100.0 ** (-2 / 8)       # position 3, pair 1: dims 1 and 5
    assert torch.allclose(y[3, 0, 1], x[3, 0, 1] * math.cos(a) - x[3, 0, 5] * math.sin(a))
    assert torch.allclose(y[3, 0, 5], x[3, 0, 5] * math.cos(a) + x[3, 0, 1] * math.sin(a))


def test_the_memory_goes_on_where_a_portion_ended_and_its_first_token_reads_itself():
    g = torch.Generator().manual_seed(1)
    T, H, dk, dv = 9, 3, 5, 4
    q, k = (torch.randn(T, H, dk, generator=g, dtype=torch.float64) for _ in range(2))
    v = torch.randn(T, H, dv, generator=g, dtype=torch.float64)
    li = torch.randn(T, H, generator=g, dtype=torch.float64) * 3
    lk = plain.log_sigmoid(torch.randn(T, H, generator=g, dtype=torch.float64) * 3)
    o, (S, n, m) = plain.matrix_memory(q, k, v, li, lk)
    o1, st = plain.matrix_memory(q[:4], k[:4], v[:4], li[:4], lk[:4])
    o2, (S2, n2, m2) = plain.matrix_memory(q[4:], k[4:], v[4:], li[4:], lk[4:], state=st)
    assert torch.allclose(torch.cat([o1, o2]), o) and torch.allclose(S2, S) and torch.allclose(n2, n) and torch.allclose(m2, m)
    # the running maximum starts at 0: a first token whose input gate is shut keeps it there
    m0 = torch.maximum(lk[0], li[0])
    take = torch.exp(li[0] - m0)
    qk = (q[0] * k[0]).sum(-1)
    want = take[:, None] * qk[:, None] * v[0] / (torch.maximum((take * qk).abs(), torch.exp(-m0)) + 1e-6)[:, None]
    assert torch.allclose(o[0], want)
    # the result does not depend on the maximum but through the floor: the same walk without it, in plain numbers
    Su = torch.zeros(H, dk, dv, dtype=torch.float64)
    nu = torch.zeros(H, dk, dtype=torch.float64)
    for t in range(T):
        Su = torch.exp(lk[t])[:, None, None] * Su + torch.exp(li[t])[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        nu = torch.exp(lk[t])[:, None] * nu + torch.exp(li[t])[:, None] * k[t]
    assert torch.allclose(S * torch.exp(m)[:, None, None], Su) and torch.allclose(n * torch.exp(m)[:, None], nu)
    assert torch.allclose(plain.log_sigmoid(torch.tensor([-50.0, 0.0, 50.0], dtype=torch.float64)),
                          torch.tensor([-50.0, -math.log(2.0), 0.0], dtype=torch.float64), atol=1e-12)


def test_the_convolution_sees_nothing_before_a_sequence():
    g = torch.Generator().manual_seed(2)
    u = torch.randn(6, 2, generator=g, dtype=torch.float64)
    w = torch.randn(2, 3, generator=g, dtype=torch.float64)
    out = plain.short_conv(u, w)
    assert torch.allclose(out[0], w[:, 2] * u[0]) and torch.allclose(out[2], w[:, 0] * u[0] + w[:, 1] * u[1] + w[:, 2] * u[2])


def test_mixed_heads_and_the_sum_on_the_querys_side():
    """Head h's mixed score is a sum over heads of talk[h, g] q_g . k_kv(g): the same number as q'_h against the token's
    whole k row, q'_h = [sum_{g on kv head c} talk[h, g] q_g for every c], which is how the engine computes it."""
    g = torch.Generator().manual_seed(3)
    T, H, G, d = 7, 6, 3, 4
    q = torch.randn(T, H, d, generator=g, dtype=torch.float64)
    k = torch.randn(T, G, d, generator=g, dtype=torch.float64)
    talk = torch.randn(H, H, generator=g, dtype=torch.float64)
    s = plain.mixed_head_scores(q, k, 0.5, talk)
    assert torch.allclose(plain.mixed_head_scores(q, k, 0.5, torch.eye(H, dtype=torch.float64))[4], (q[:, 4] @ k[:, 2].T) * 0.5)
    folded = torch.zeros(T, H, G, d, dtype=torch.float64)
    for h in range(H):
        for j in range(H):
            folded[:, h, j // (H // G)] += talk[h, j] * q[:, j]
    again = torch.einsum("ihx,jx->hij", folded.reshape(T, H, G * d), k.reshape(T, G * d)) * 0.5
    assert torch.allclose(s, again)


def test_an_expert_sees_the_token_times_its_score():
    g = torch.Generator().manual_seed(4)
    h = torch.randn(3, 8, generator=g, dtype=torch.float64)
    w = {"router": torch.randn(2, 8, generator=g, dtype=torch.float64)}
    for e in range(2):
        w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"] = (torch.randn(*s, generator=g, dtype=torch.float64) for s in ((5, 8), (5, 8), (8, 5)))
    out = plain.routed_experts(h, w, {"router": {"experts": 2, "top": 1}})
    s = torch.sigmoid(h @ w["router"].T)
    e = int(s[1].argmax())
    x = h[1] * s[1, e]
    assert torch.allclose(out[1], (plain.silu(w[f"e{e}.gate"] @ x) * (w[f"e{e}.up"] @ x)) @ w[f"e{e}.down"].T)
    both = plain.routed_experts(h, w, {"router": {"experts": 2, "top": 2}})
    assert not torch.allclose(both, out)
