"""Rukedra without a GPU: the configuration reader, the rotation tables, where checkpoint tensors land in the fused input
projections and the stacked experts, layers that borrow weights, and the oracle's own mechanisms on hand-made inputs."""

import math

import pytest
import torch

from tests import _layered as L
from tests import _rukedra as T


def _geometry(cfg):
    from lite_llama_amd.model_layers import LayeredGeometry

    return LayeredGeometry.from_config(cfg, name="rukedra")


def test_reader_takes_every_size_and_constant_from_the_configuration():
    geo = _geometry(T.CONFIGS["mix"])
    assert geo.sandwich and not geo.token_shift and geo.norm_groups == 3 and geo.logit_softcap == 9.0 and geo.width == 96
    kinds = [s.mixer.kind for s in geo.layers]
    assert kinds == ["mingru", "latent_attention", "latent_attention", "latent_attention", "latent_attention"]
    a, b = geo.layers[1].mixer, geo.layers[2].mixer
    assert (a.heads, a.dim, a.rot_dim, a.vdim, a.kv_rank, a.q_rank, a.window, a.out_gate) == (3, 24, 8, 16, 40, 24, 9, True)
    assert (b.heads, b.dim, b.rot_dim, b.vdim, b.kv_rank, b.q_rank, b.window, b.out_gate) == (2, 16, 16, 24, 24, 0, 0, False)
    assert geo.layers[3].weights_of == 1 and geo.layers[3].mixer == geo.layers[1].mixer and geo.layers[2].mlp is None
    m = geo.layers[0].mlp
    assert (m.kind, m.experts, m.top, m.group_count, m.group_keep, m.route_scale, m.shared_ff, m.ff) == ("moe", 6, 3, 3, 2, 2.0, 40, 24)
    m = geo.layers[4].mlp
    assert (m.group_count, m.group_keep, m.shared_ff) == (1, 1, 0)
    assert _geometry(T.CONFIGS["odd"]).logit_softcap == 0.0


@pytest.mark.parametrize("bad", ["type", "groups", "borrow", "top", "rot"])
def test_reader_refuses_what_it_cannot_build(bad):
    import copy

    cfg = copy.deepcopy(T.CONFIGS["mix"])
    if bad == "type":
        cfg["layers"][0]["type"] = "lstm"
    elif bad == "groups":
        cfg["norm"]["groups"] = 5
    elif bad == "borrow":
        cfg["layers"][4]["weights_of"] = 3                          # layer 3 borrows itself: it owns nothing
    elif bad == "top":
        cfg["layers"][0]["mlp"]["router"]["groups"]["keep"] = 1     # one group of two experts cannot give three
    else:
        cfg["layers"][1]["mixer"]["rot"]["dims"] = 10
    with pytest.raises(ValueError):
        _geometry(cfg)


@pytest.mark.parametrize("kw", [dict(dims=8), dict(dims=16, base=10000.0, factor=8.0, original=40, fast=8.0, slow=1.0),
                                dict(dims=6, base=37.0, factor=2.5, original=24), dict(dims=4, factor=8.0, original=16, fast=2.0)])
def test_rotation_table_equals_the_oracle(kw):
    from lite_llama_amd.model_layers import RotarySpec
    from oracle import rukedra as O

    desc = T.rot(**kw)
    freq, amp = RotarySpec.from_config(desc).table()
    want, want_amp = O.yarn_frequencies(desc)
    assert amp == pytest.approx(want_amp, rel=1e-12) and amp == pytest.approx(0.1 * math.log(desc["scaling"]["factor"]) + 1)
    assert torch.allclose(torch.tensor(freq, dtype=torch.float64), want, rtol=1e-12, atol=0)
    plain = RotarySpec(dims=8, base=100.0).table()
    assert plain[1] == 1.0 and plain[0] == pytest.approx([100.0 ** (-i / 4) for i in range(4)])
    # the two ends of the ramp: the fastest pair keeps its frequency, the slowest is divided by the factor
    if kw["dims"] == 16:
        assert freq[0] == pytest.approx(1.0) and freq[-1] == pytest.approx(10000.0 ** (-14 / 16) / 8.0)


@pytest.mark.parametrize("name", sorted(T.CONFIGS))
def test_checkpoint_lands_in_the_fused_projections_and_borrowed_layers_share_modules(tmp_path, name):
    from lite_llama_amd.weights import load_pretrained

    cfg = T.CONFIGS[name]
    tens = T.tensors(cfg, seed=3)
    model = load_pretrained(L.write(tmp_path, cfg, tens), device="cpu", dtype=torch.float32)
    W = cfg["width"]
    assert len(model.cache_runs()) == len(cfg["layers"])
    for i, entry in enumerate(cfg["layers"]):
        layer, p = model.layers[i], f"l{entry.get('weights_of', i)}."
        if entry.get("weights_of") is not None:
            assert layer is model.layers[entry["weights_of"]]          # (the owner may come later in the stack)
            continue
        w = layer.mixer.in_proj.weight
        assert torch.equal(w[-W:], tens[p + "rg1"]) and torch.equal(layer.rg1_bias, tens[p + "rg1.b"])
        m = entry["mixer"]
        if entry["type"] == "mingru":
            n = m["width"]
            assert torch.equal(w[:n], tens[p + "mix.z"]) and torch.equal(w[n:2 * n], tens[p + "mix.x"]) and torch.equal(w[2 * n:3 * n], tens[p + "mix.g"])
        else:
            q = m.get("q_rank") or m["heads"] * (m["dim"] + m["rot_dim"])
            assert torch.equal(w[:q], tens[p + ("mix.dq" if "q_rank" in m else "mix.q")])
            assert torch.equal(w[q:q + m["kv_rank"] + m["rot_dim"]], tens[p + "mix.dkv"])
            if entry["type"] == "latent_attention":
                assert torch.equal(w[q + m["kv_rank"] + m["rot_dim"]:-W], tens[p + "mix.g"])
            assert torch.equal(layer.mixer.uk_weight, tens[p + "mix.uk"])
        mlp = entry["mlp"]
        if mlp is None:
            assert layer.mlp is None
        elif mlp["kind"] == "dense":
            assert torch.equal(layer.mlp.in_proj.weight, torch.cat([tens[p + "mlp.gate"], tens[p + "mlp.up"], tens[p + "rg2"]]))
        else:
            ff = mlp["expert"]["ff"]
            for e in range(mlp["router"]["experts"]):
                assert torch.equal(layer.mlp.gate_up_weight[e, :ff], tens[f"{p}mlp.e{e}.gate"])
                assert torch.equal(layer.mlp.gate_up_weight[e, ff:], tens[f"{p}mlp.e{e}.up"])
                assert torch.equal(layer.mlp.down_weight[e], tens[f"{p}mlp.e{e}.down"])
            assert torch.equal(layer.mlp.in_proj.weight[-W:], tens[p + "rg2"])
    # a missing and an unknown tensor are both named
    short = dict(tens)
    owner = next(i for i, e in enumerate(cfg["layers"]) if e.get("weights_of") is None)
    del short[f"l{owner}.rg1.b"]
    with pytest.raises(ValueError, match="rg1_bias"):
        load_pretrained(L.write(tmp_path / "short", cfg, short), device="cpu", dtype=torch.float32)
    with pytest.raises(ValueError, match="unknown parameter"):
        load_pretrained(L.write(tmp_path / "more", cfg, dict(tens, **{"l0.mix.sink": torch.zeros(2)})), device="cpu", dtype=torch.float32)


# ------------------------------------------------------------------------------------------------------------------- #
# the oracle on inputs whose answer is known by hand
# ------------------------------------------------------------------------------------------------------------------- #
def test_oracle_group_norm_and_router_on_hand_made_inputs():
    from oracle import rukedra as O

    x = torch.tensor([[3.0, 4.0, 0.0, 10.0]], dtype=torch.float64)
    got = O.group_rms_norm(x, torch.ones(4, dtype=torch.float64), 0.0, 2)
    assert torch.allclose(got, torch.tensor([[3 / math.sqrt(12.5), 4 / math.sqrt(12.5), 0.0, math.sqrt(2.0)]], dtype=torch.float64))
    # six experts in three pairs; logits make pair 1 the best group by the SUM of its two, although expert 4 is the best single
    logits = torch.tensor([[0.0, 0.1, 1.0, 1.1, 2.0, -1.0]], dtype=torch.float64)
    router = {"experts": 6, "top": 2, "scale": 3.0, "groups": {"count": 3, "keep": 1}}
    idx, w = O.route(logits, torch.eye(6, dtype=torch.float64), router)
    assert idx.tolist() == [[3, 2]]
    s = torch.sigmoid(logits[0, [3, 2]])
    assert torch.allclose(w[0], s / s.sum() * 3.0)
    idx, _ = O.route(logits, torch.eye(6, dtype=torch.float64), dict(router, groups={"count": 3, "keep": 2}))
    assert idx.tolist() == [[4, 3]]


def test_oracle_window_and_rotation_on_hand_made_inputs():
    from oracle import rukedra as O

    v = torch.tensor([[1.0, 0.0, 5.0]], dtype=torch.float64)
    desc = {"base": 100.0, "dims": 2}
    out = O.rotate_pairs(v.repeat(3, 1), torch.tensor([0, 1, 2]), desc)
    assert torch.allclose(out[:, 0], torch.cos(torch.tensor([0.0, 1.0, 2.0], dtype=torch.float64)))
    assert torch.allclose(out[:, 1], torch.sin(torch.tensor([0.0, 1.0, 2.0], dtype=torch.float64))) and torch.all(out[:, 2] == 5.0)
    # minGRU with z = 1/2 and candidate 1 from a zero state: 1/2, 3/4, 7/8
    w = {"z": torch.zeros(1, 1), "z.b": torch.zeros(1), "x": torch.zeros(1, 1), "x.b": torch.full((1,), 0.5), "g": torch.zeros(1, 1),
         "o": torch.ones(1, 1)}
    w = {k: t.double() for k, t in w.items()}
    w["g"], h = torch.ones(1, 1, dtype=torch.float64), torch.ones(3, 1, dtype=torch.float64)
    got = O.mingru(h, w, "")
    silu1 = 1 / (1 + math.exp(-1.0))
    assert torch.allclose(got[:, 0], torch.tensor([0.5, 0.75, 0.875], dtype=torch.float64) * silu1)
