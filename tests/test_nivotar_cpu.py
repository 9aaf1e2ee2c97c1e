"""Nivotar without a GPU: the configuration reader (with the one size that only a tensor's shape gives), where checkpoint
tensors land in the fused input / output projections, the bias vectors and the stacked experts, what the cache manager is asked
to set up for the design, and the oracle's own mechanisms on hand-made inputs."""

import copy
import math

import pytest
import torch

from tests import _layered as L
from tests import _nivotar as T


def _folder(tmp_path, name, seed=0):
    cfg = T.CONFIGS[name]
    tens = T.tensors(cfg, seed=seed)
    return L.write(tmp_path / name, T.on_disk(cfg), tens), T.on_disk(cfg), tens


def _geometry(cfg, shapes=None):
    from lite_llama_amd.model_layers import LayeredGeometry

    return LayeredGeometry.from_config(cfg, name="nivotar", shapes=shapes)


def test_reader_takes_every_size_and_constant_from_the_configuration_and_the_rank_from_a_shape(tmp_path):
    from lite_llama_amd.weights import tensor_shapes

    folder, cfg, _ = _folder(tmp_path, "mix")
    geo = _geometry(cfg, tensor_shapes(folder))
    assert geo.post_norm and geo.tied_head and not (geo.sandwich or geo.parallel or geo.token_shift) and (geo.width, geo.vocab_size) == (96, 83)
    a, b, c, e = (layer.mixer for layer in geo.layers)
    assert a.kind == "attention_ssd" and (a.heads, a.kv_heads, a.dim, a.vdim, a.window) == (4, 2, 16, 8, 9)
    assert a.rotary.dims == 8 and a.rotary.base == 100.0 and a.rotary.factor == 0.0 and a.scale == pytest.approx(0.5)
    assert (a.ssd.heads, a.ssd.vdim, a.ssd.state, a.ssd.groups, a.ssd.conv_taps, a.ssd.norm_groups) == (4, 8, 16, 2, 4, 2)
    assert a.branch_scales == (0.7, 1.2) and a.ssd.inner == 32 and a.ssd.conv_channels == 96
    assert b.kind == "decay_linear" and b.decay == (0.8, 0.995) and (b.heads, b.dim, b.vdim) == (2, 16, 24)
    assert c.kind == "gla" and (c.heads, c.dim, c.vdim, c.tau, c.decay_rank) == (3, 16, 8, 8.0, 8)
    assert e.window == 21 and e.ssd.groups == 1
    d0, d1, d2 = geo.layers[0].mlp, geo.layers[1].mlp, geo.layers[2].mlp
    assert (d0.kind, d0.ff, d0.act, d0.bias) == ("dense", 72, "silu", True) and geo.layers[3].mlp is None
    assert (d1.kind, d1.experts, d1.identity, d1.top, d1.ff, d1.limit, d1.scoring) == ("moe", 6, 2, 3, 24, 2.5, "softmax_all")
    assert d2.limit == 0.75 and d2.identity == 1
    with pytest.raises(ValueError):
        _geometry(cfg)                     # (without the shapes the rank of the decay projection is unknown)


@pytest.mark.parametrize("bad", ["type", "heads", "rot", "odd_rot", "top", "kind", "decay", "groups", "parts"])
def test_reader_refuses_what_it_cannot_build(bad):
    cfg = copy.deepcopy(T.on_disk(T.CONFIGS["mix"]))
    if bad == "type":
        cfg["layers"][0]["type"] = "lstm"
    elif bad == "heads":
        cfg["layers"][0]["mixer"]["left"]["kv_heads"] = 3
    elif bad == "rot":
        cfg["layers"][0]["mixer"]["left"]["rot"]["dims"] = 18
    elif bad == "odd_rot":
        cfg["layers"][0]["mixer"]["left"]["rot"]["dims"] = 7
    elif bad == "top":
        cfg["layers"][1]["mlp"]["router"]["top"] = 9
    elif bad == "kind":
        cfg["layers"][0]["mlp"]["kind"] = "conv"
    elif bad == "decay":
        cfg["layers"][1]["mixer"]["decay"] = [0.5]
    elif bad == "groups":
        cfg["layers"][0]["mixer"]["right"]["groups"] = 3
    else:
        cfg["layers"][0]["mixer"]["right"]["norm_groups"] = 5
    with pytest.raises(ValueError):
        _geometry(cfg, {"l2.mix.a1": (8, 96)})


@pytest.mark.parametrize("name", sorted(T.CONFIGS))
def test_checkpoint_lands_in_the_fused_projections(tmp_path, name):
    from lite_llama_amd.weights import load_pretrained

    folder, cfg, tens = _folder(tmp_path, name, seed=3)
    model = load_pretrained(folder, device="cpu", dtype=torch.float32)
    assert model.lm_head.weight is model.embed_tokens.weight and torch.equal(model.embed_tokens.weight, tens["embed"])
    for i, entry in enumerate(cfg["layers"]):
        layer, p, m = model.layers[i], f"l{i}.", entry["mixer"]
        w = layer.mixer.in_proj.weight
        if entry["type"] == "parallel":
            a, r = m["left"], m["right"]
            q, k, v = a["heads"] * a["dim"], a["kv_heads"] * a["dim"], a["kv_heads"] * a["vdim"]
            assert torch.equal(w[:q], tens[p + "mix.left.q"]) and torch.equal(w[q:q + k], tens[p + "mix.left.k"])
            assert torch.equal(w[q + k:q + k + v], tens[p + "mix.left.v"]) and torch.equal(w[q + k + v:], tens[p + "mix.right.in"])
            hw = a["heads"] * a["vdim"]
            assert torch.equal(layer.mixer.out_proj.weight[:, :hw], tens[p + "mix.left.o"])
            assert torch.equal(layer.mixer.out_proj.weight[:, hw:], tens[p + "mix.right.o"])
            assert torch.equal(layer.mixer.skip, tens[p + "mix.right.D"]) and torch.equal(layer.mixer.a_log, tens[p + "mix.right.A_log"])
            assert torch.equal(layer.mixer.conv_weight, tens[p + "mix.right.conv"])
            run = layer.mixer.cache_run()
            assert run["kind"] == "attention" and run["state"] == (r["heads"], r["state"], r["vdim"])
            assert (run["conv_taps"], run["conv_channels"]) == (r["conv"], r["heads"] * r["vdim"] + 2 * r["groups"] * r["state"])
        else:
            qk, v = m["heads"] * m["dim"], m["heads"] * m["vdim"]
            assert torch.equal(w[:qk], tens[p + "mix.q"]) and torch.equal(w[qk:2 * qk], tens[p + "mix.k"])
            assert torch.equal(w[2 * qk:2 * qk + v], tens[p + "mix.v"]) and torch.equal(w[2 * qk + v:2 * qk + 2 * v], tens[p + "mix.g"])
            if entry["type"] == "gla":
                assert torch.equal(w[2 * qk + 2 * v:], tens[p + "mix.a1"]) and torch.equal(layer.mixer.decay_proj.weight, tens[p + "mix.a2"])
                assert torch.equal(layer.mixer.decay_bias, tens[p + "mix.a2.b"])
            else:
                assert w.shape[0] == 2 * qk + 2 * v
            assert layer.mixer.cache_run() == {"kind": "recurrent", "heads": m["heads"], "dk": m["dim"], "dv": m["vdim"]}
        mlp = entry["mlp"]
        if mlp is None:
            assert layer.mlp is None
        elif mlp["kind"] == "dense":
            ff = mlp["ff"]
            assert torch.equal(layer.mlp.in_proj.weight[:ff], tens[p + "mlp.gate"]) and torch.equal(layer.mlp.in_proj.weight[ff:], tens[p + "mlp.up"])
            assert torch.equal(layer.mlp.in_proj.bias[:ff], tens[p + "mlp.gate.b"]) and torch.equal(layer.mlp.in_proj.bias[ff:], tens[p + "mlp.up.b"])
            assert torch.equal(layer.mlp.down_bias, tens[p + "mlp.down.b"])
        else:
            ff = mlp["expert"]["ff"]
            for e in range(mlp["router"]["experts"]):
                assert torch.equal(layer.mlp.gate_up_weight[e, :ff], tens[f"{p}mlp.e{e}.gate"])
                assert torch.equal(layer.mlp.gate_up_weight[e, ff:], tens[f"{p}mlp.e{e}.up"])
                assert torch.equal(layer.mlp.down_weight[e], tens[f"{p}mlp.e{e}.down"])
            assert layer.mlp.router_weight.shape[0] == mlp["router"]["experts"] + mlp["router"]["identity"]
            assert torch.equal(layer.mlp.correction, tens[p + "mlp.correction"])


def test_loader_names_missing_and_unknown_tensors(tmp_path):
    from lite_llama_amd.weights import load_pretrained

    cfg = T.CONFIGS["mix"]
    tens = T.tensors(cfg)
    missing = dict(tens)
    del missing["l0.mix.right.dt_bias"]
    with pytest.raises(ValueError, match="dt_bias"):
        load_pretrained(L.write(tmp_path / "a", T.on_disk(cfg), missing), device="cpu", dtype=torch.float32)
    extra = dict(tens, **{"l1.mix.sink": torch.zeros(2)})
    with pytest.raises(ValueError, match="sink"):
        load_pretrained(L.write(tmp_path / "b", T.on_disk(cfg), extra), device="cpu", dtype=torch.float32)


def test_the_trace_replay_and_the_engine_know_the_family():
    from lite_llama_amd.weights import MODEL_FAMILIES, model_family

    assert model_family({"architecture": "Nivotar"}) == "nivotar" and "nivotar" in MODEL_FAMILIES


# ------------------------------------------------------------------------------------------------------------------- #
# the oracle's mechanisms on inputs small enough to do by hand
# ------------------------------------------------------------------------------------------------------------------- #
def test_oracle_rotation_pairs_entry_i_with_entry_i_plus_half():
    from oracle import nivotar as O

    x = torch.zeros(2, 1, 6, dtype=torch.float64)
    x[:, 0, 0], x[:, 0, 3], x[:, 0, 4], x[:, 0, 5] = 1.0, 2.0, 5.0, 7.0
    y = O.rotate_half(x, torch.tensor([0, 3]), 4, 100.0)         # pairs (0, 2) and (1, 3); entries 4, 5 pass
    assert torch.equal(y[0], x[0])
    a0, a1 = 3.0, 3.0 * 100.0 ** -0.5
    want = [math.cos(a0), -2.0 * math.sin(a1), math.sin(a0), 2.0 * math.cos(a1), 5.0, 7.0]
    assert torch.allclose(y[1, 0], torch.tensor(want, dtype=torch.float64), atol=1e-12)


def test_oracle_window_sees_itself_and_size_minus_one_before():
    from oracle import nivotar as O

    m = O.visible(6, 3)
    assert m[5].tolist() == [False, False, False, True, True, True] and m[1].tolist() == [True, True, False, False, False, False]
    assert O.visible(4, 1).int().sum().item() == 4


def test_oracle_convolution_ends_at_the_current_token_and_starts_from_zeros():
    from oracle import nivotar as O

    u = torch.tensor([[1.0], [10.0], [100.0]], dtype=torch.float64)
    y = O.causal_conv(u, torch.tensor([[3.0, 2.0, 1.0]], dtype=torch.float64), torch.tensor([0.5], dtype=torch.float64))
    assert y[:, 0].tolist() == [1.5, 12.5, 123.5]                  # the last column weighs the current token


def test_oracle_decaying_state_by_hand():
    from oracle import nivotar as O

    q = torch.tensor([[1.0, 0.0], [1.0, 1.0]], dtype=torch.float64)
    k = torch.tensor([[2.0, 1.0], [0.0, 1.0]], dtype=torch.float64)
    v = torch.tensor([[1.0], [3.0]], dtype=torch.float64)
    a = torch.tensor([[0.5, 0.25], [0.5, 0.25]], dtype=torch.float64)
    o, S = O.decay_scan(q, k, v, a)
    assert o[:, 0].tolist() == [2.0, 1.0 + 0.25 + 3.0] and S[:, 0].tolist() == [1.0, 3.25]


def test_oracle_router_corrects_the_choice_not_the_weight_and_identity_returns_the_input():
    from oracle import nivotar as O

    t = {"router": torch.tensor([[2.0], [1.0], [0.0]], dtype=torch.float64), "correction": torch.tensor([0.0, -1.0, 1.0], dtype=torch.float64),
         "e0.gate": torch.ones(1, 1, dtype=torch.float64), "e0.up": torch.ones(1, 1, dtype=torch.float64), "e0.down": torch.ones(1, 1, dtype=torch.float64),
         "e1.gate": torch.ones(1, 1, dtype=torch.float64), "e1.up": torch.ones(1, 1, dtype=torch.float64), "e1.down": torch.ones(1, 1, dtype=torch.float64)}
    x = torch.tensor([[1.0]], dtype=torch.float64)
    ids, w = O.route(x, t, "", {"top": 2})
    s = torch.softmax(torch.tensor([2.0, 1.0, 0.0], dtype=torch.float64), 0)
    assert ids[0].tolist() == [2, 0] and torch.allclose(w[0], s[[2, 0]])          # output 1 outscores 2, the correction turns it
    mlp = {"router": {"experts": 2, "identity": 1, "top": 2}, "expert": {"limit": 0.5}}
    y = O.moe(x, t, "", mlp)
    g = 0.5                                                                        # the gate is clamped from 1 to 0.5, up too
    expert = g / (1 + math.exp(-1.702 * g)) * (0.5 + 1.0)
    assert torch.allclose(y, s[2] * x + s[0] * expert)
