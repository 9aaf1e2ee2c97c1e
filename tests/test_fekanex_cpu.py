"""Fekanex without a GPU: the configuration reader, where checkpoint tensors land in the fused input / output projections, the
bias vector, the tap matrix and the stacked experts, what the cache manager sets up for the design, and the oracle's own
mechanisms on hand-made inputs."""

import copy
import math

import pytest
import torch

from tests import _fekanex as T
from tests import _layered as L


def _geometry(cfg):
    from lite_llama_amd.model_layers import LayeredGeometry

    return LayeredGeometry.from_config(cfg, name="fekanex")


def test_reader_takes_every_size_and_constant_from_the_configuration():
    geo = _geometry(T.CONFIGS["mix"])
    assert geo.parallel and not geo.sandwich and not geo.token_shift and geo.tied_head and geo.width == 96 and geo.vocab_size == 83
    assert (geo.embed_scale, geo.pair_buckets, geo.pair_mul_prev, geo.pair_mul_cur, geo.logit_scale) == (0.25, 31, 7, 3, 3.0)
    a, c = geo.layers[0].mixer, geo.layers[2].mixer
    assert a.kind == "conv_attention" and a.bias and a.unit_norm and a.unit_sink
    assert (a.heads, a.kv_heads, a.dim, a.vdim, a.conv_taps, a.window, a.keep_first, a.value_mix) == (4, 2, 16, 8, 4, 9, 3, True)
    assert (c.heads, c.kv_heads, c.dim, c.vdim, c.conv_taps, c.window, c.keep_first, c.value_mix) == (2, 1, 24, 16, 2, 5, 0, False)
    assert a.rotary.dims == 8 and c.rotary.dims == 24 and c.rotary.base == 37.0 and c.rotary.factor == 2.5
    assert a.scale == pytest.approx(3.0 / 4.0)
    d, e = geo.layers[0].mlp, geo.layers[3].mlp
    assert (d.kind, d.ff, d.act, d.limit) == ("dense", 72, "clamped", 1.5) and geo.layers[2].mlp is None
    assert (e.kind, e.experts, e.top, e.ff, e.scoring) == ("moe", 4, 4, 16, "softmax_chosen")
    odd = _geometry(T.CONFIGS["odd"])
    assert odd.layers[0].mixer.rotary.factor == 0.0 and odd.layers[2].mixer.conv_taps == 0 and odd.layers[1].mixer.conv_taps == 1
    assert odd.eps == 1e-6 and odd.logit_scale == 0.5 and odd.layers[0].mlp.limit == 0.75
    assert len(geo.run_order()) == 4


@pytest.mark.parametrize("bad", ["type", "heads", "rot", "odd_rot", "top", "kind"])
def test_reader_refuses_what_it_cannot_build(bad):
    cfg = copy.deepcopy(T.CONFIGS["mix"])
    if bad == "type":
        cfg["layers"][0]["type"] = "lstm"
    elif bad == "heads":
        cfg["layers"][0]["mixer"]["kv_heads"] = 3
    elif bad == "rot":
        cfg["layers"][1]["mixer"]["rot"]["dims"] = 18
    elif bad == "odd_rot":
        cfg["layers"][1]["mixer"]["rot"]["dims"] = 7
    elif bad == "top":
        cfg["layers"][1]["mlp"]["router"]["top"] = 7
    else:
        cfg["layers"][0]["mlp"]["kind"] = "conv"
    with pytest.raises(ValueError):
        _geometry(cfg)


@pytest.mark.parametrize("name", sorted(T.CONFIGS))
def test_checkpoint_lands_in_the_fused_projections(tmp_path, name):
    from lite_llama_amd.weights import load_pretrained

    cfg = T.CONFIGS[name]
    tens = T.tensors(cfg, seed=3)
    model = load_pretrained(L.write(tmp_path / name, cfg, tens), device="cpu", dtype=torch.float32)
    assert model.lm_head.weight is model.embed_tokens.weight and torch.equal(model.embed_tokens.weight, tens["embed"])
    assert torch.equal(model.pair_table, tens["bigram"]) and model.needs_previous_token
    names = [n for n, _ in model.named_parameters()]
    assert not any(n.startswith("lm_head") for n in names)
    for i, entry in enumerate(cfg["layers"]):
        layer, m, p = model.layers[i], entry["mixer"], f"l{i}."
        q, k, v = m["heads"] * m["dim"], m["kv_heads"] * m["dim"], m["kv_heads"] * m["vdim"]
        w_in, hw = layer.mixer.in_proj.weight, m["heads"] * m["vdim"]
        at = 0
        for leaf, rows in (("q", q), ("k", k), ("v", v)):
            assert torch.equal(w_in[at:at + rows], tens[p + "mix." + leaf])
            assert torch.equal(layer.mixer.qkv_bias[at:at + rows], tens[p + "mix." + leaf + ".b"])
            if m.get("conv"):
                assert torch.equal(layer.mixer.conv_weight[at:at + rows], tens[p + "mix." + leaf + ".conv"])
            at += rows
        assert (layer.mixer.conv_weight is None) == (not m.get("conv"))
        assert torch.equal(layer.out_proj.weight[:, :hw], tens[p + "mix.o"])
        if m["v_mix"]:
            assert layer.mixer.value_blend.shape == (1,) and layer.mixer.value_blend[0] == tens[p + "mix.vmix"]
        else:
            assert layer.mixer.value_blend is None
        mlp = entry["mlp"]
        if mlp is None:
            assert w_in.shape[0] == at and layer.out_proj.weight.shape[1] == hw and layer.experts is None
        elif mlp["kind"] == "dense":
            ff = mlp["ff"]
            assert torch.equal(w_in[at:at + ff], tens[p + "mlp.gate"]) and torch.equal(w_in[at + ff:], tens[p + "mlp.up"])
            assert torch.equal(layer.out_proj.weight[:, hw:], tens[p + "mlp.down"]) and layer.experts is None
        else:
            ff = mlp["expert"]["ff"]
            assert w_in.shape[0] == at and torch.equal(layer.experts.router_weight, tens[p + "mlp.router"])
            for e in range(mlp["router"]["experts"]):
                assert torch.equal(layer.experts.gate_up_weight[e, :ff], tens[f"{p}mlp.e{e}.gate"])
                assert torch.equal(layer.experts.gate_up_weight[e, ff:], tens[f"{p}mlp.e{e}.up"])
                assert torch.equal(layer.experts.down_weight[e], tens[f"{p}mlp.e{e}.down"])


def test_loader_names_missing_and_unknown_tensors(tmp_path):
    from lite_llama_amd.weights import load_pretrained

    cfg = T.CONFIGS["odd"]
    tens = T.tensors(cfg)
    missing = {k: v for k, v in tens.items() if k != "l1.mix.k.b"}
    with pytest.raises(ValueError, match="qkv_bias"):
        load_pretrained(L.write(tmp_path / "a", cfg, missing), device="cpu", dtype=torch.float32)
    with pytest.raises(ValueError, match="l2.mix.q.conv"):     # a layer without a convolution has no taps
        load_pretrained(L.write(tmp_path / "b", cfg, dict(tens, **{"l2.mix.q.conv": torch.zeros(40, 2)})), device="cpu",
                        dtype=torch.float32)
    # a blend weight of a layer that does not blend is passed over
    load_pretrained(L.write(tmp_path / "c", cfg, dict(tens, **{"l0.mix.vmix": torch.tensor(0.5)})), device="cpu", dtype=torch.float32)


def test_family_is_registered_and_the_cache_sets_up_carried_rows_previous_tokens_and_value_sources():
    from lite_llama_amd.model_layers import LayeredLM
    from lite_llama_amd.weights import MODEL_FAMILIES, model_family

    cfg = T.CONFIGS["odd"]
    assert model_family(cfg) == "fekanex" and "fekanex" in MODEL_FAMILIES
    runs = LayeredLM(_geometry(cfg), dtype=torch.float32).cache_runs()
    assert [r["kind"] for r in runs] == ["attention"] * 4
    assert [r["conv_taps"] for r in runs] == [3, 1, 0, 5] and [r["value_mix"] for r in runs] == [False, True, True, True]
    assert runs[0]["conv_channels"] == 5 * 12 + 5 * 12 + 5 * 10 and (runs[3]["kv_heads"], runs[3]["dk"], runs[3]["dv"]) == (1, 12, 10)


def test_oracle_pair_rows_convolution_and_mask_on_hand_made_inputs():
    from oracle import fekanex as O

    assert O.bigram_rows([4, 9, 9, 0], {"buckets": 7, "mul_prev": 3, "mul_cur": 5}) == [7, (12 + 45) % 7, (27 + 45) % 7, 27 % 7]
    assert O.bigram_rows([2], {"buckets": 1, "mul_prev": 3, "mul_cur": 5}) == [1]
    u = torch.tensor([[1.0, 10.0], [2.0, 20.0], [3.0, 30.0], [4.0, 40.0]], dtype=torch.float64)
    w = torch.tensor([[100.0, 10.0, 1.0], [0.0, 0.0, 2.0]], dtype=torch.float64)    # the LAST tap meets the token itself
    y = O.causal_conv(u, w)
    assert y[:, 0].tolist() == [1.0, 12.0, 123.0, 234.0] and y[:, 1].tolist() == [20.0, 40.0, 60.0, 80.0]
    assert torch.equal(O.causal_conv(u, torch.tensor([[2.0], [3.0]], dtype=torch.float64)), u * torch.tensor([2.0, 3.0]))
    seen = O.visible(7, 2, 3)
    assert seen[6].tolist() == [True, True, True, False, False, True, True]
    assert seen[3].tolist() == [True, True, True, True, False, False, False]
    assert O.visible(4, 5, 0)[3].tolist() == [True] * 4 and O.visible(4, 1, 0)[3].tolist() == [False, False, False, True]


def test_oracle_softmax_with_a_unit_sink_rotation_feed_forward_and_routing_on_hand_made_inputs():
    from oracle import fekanex as O

    s = torch.tensor([[0.0, math.log(3.0), 5.0]], dtype=torch.float64)
    w = O.sink_softmax(s, torch.tensor([[True, True, False]]))
    assert torch.allclose(w, torch.tensor([[0.2, 0.6, 0.0]], dtype=torch.float64))        # 1 / (1 + 1 + 3), 3 / 5: the sink keeps 1 / 5
    big = O.sink_softmax(torch.tensor([[800.0, -800.0]], dtype=torch.float64), torch.tensor([[True, True]]))
    assert torch.allclose(big, torch.tensor([[1.0, 0.0]], dtype=torch.float64)) and torch.isfinite(big).all()
    v = torch.tensor([[[1.0, 0.0, 5.0, 7.0]], [[1.0, 0.0, 5.0, 7.0]]], dtype=torch.float64)
    r = O.rotate_pairs(v, torch.tensor([0, 1]), {"dims": 2, "base": 10.0})
    assert torch.allclose(r[0], v[0]) and torch.allclose(r[1, 0], torch.tensor([math.cos(1.0), math.sin(1.0), 5.0, 7.0], dtype=torch.float64))
    f, amp = O.yarn_frequencies({"dims": 4, "base": 100.0, "scaling": {"factor": 4.0, "original": 64, "fast": 4.0, "slow": 0.5}})
    assert amp == pytest.approx(0.1 * math.log(4.0) + 1.0) and float(f[0]) == pytest.approx(1.0) and float(f[1]) == pytest.approx(0.1 / 4.0 * 0.5 + 0.1 * 0.5)   # (ramp 1 / 2: lo = 0, hi = 2)
    eye = torch.eye(2, dtype=torch.float64)
    t = {"gate": eye, "up": eye, "down": eye}
    y = O.clamped_glu(torch.tensor([[9.0, -9.0], [1.0, 0.5]], dtype=torch.float64), t, "", 2.0)
    sg = lambda z: 1 / (1 + math.exp(-1.702 * z))   # noqa: E731
    assert torch.allclose(y, torch.tensor([[2.0 * sg(2.0) * 3.0, -9.0 * sg(-9.0) * (-2.0 + 1.0)], [sg(1.0) * 2.0, 0.5 * sg(0.5) * 1.5]],
                                          dtype=torch.float64))
    ids, wts = O.route(torch.tensor([[1.0, 0.0]], dtype=torch.float64), torch.tensor([[0.5, 0], [3.0, 0], [2.0, 0], [-1.0, 0]], dtype=torch.float64), 2)
    assert ids.tolist() == [[1, 2]] and torch.allclose(wts, torch.softmax(torch.tensor([[3.0, 2.0]], dtype=torch.float64), -1))


def test_oracle_blends_values_with_the_first_blending_layer_only():
    """Layer 0 of the odd configuration does not blend: changing ITS values' projection must leave no trace in what layer 1,
    the first blending layer, hands to the later ones other than through the residual stream."""
    from oracle import fekanex as O

    cfg = T.CONFIGS["odd"]
    tens = T.tensors(cfg, seed=1)
    toks = L.prompt(cfg, 12)
    base = O.forward(toks, tens, cfg)
    changed = dict(tens, **{"l2.mix.vmix": torch.tensor(0.0)})
    assert not torch.allclose(O.forward(toks, changed, cfg), base)
    first = dict(tens, **{"l1.mix.vmix": torch.tensor(0.9)})       # the first blending layer's own weight is unused
    assert torch.equal(O.forward(toks, first, cfg), base)
