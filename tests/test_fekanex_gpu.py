"""Fekanex on the GPU against the plain CPU restatement (oracle/fekanex.py): each mechanism's kernels alone, then whole models
built from small random checkpoints through the loader, the ragged runner, the paged state cache, the generation engine and
the command line.  float32 runs are held to rounding error; bfloat16 runs to the rounding of their activations.  Where random
weights would hide a fault (a kept first key far back, a window's edge, the sink), one key is made to dominate."""

import json
import os
import subprocess
import sys

import pytest
import torch

from tests import _fekanex as T
from tests import _layered as L
from tests.test_layered_gpu import _close, _feed, _step

pytestmark = pytest.mark.gpu
DEV = "cuda"
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
F64 = torch.float64
TOL = {torch.float32: 2e-5, torch.bfloat16: 2e-2}


def d(t):
    return t.detach().cpu().to(F64)


# ------------------------------------------------------------------------------------------------------------------- #
# mechanisms alone
# ------------------------------------------------------------------------------------------------------------------- #
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width,buckets,mp,mc,scale", [(72, 31, 7, 3, 0.5), (70, 1, 3, 5, 2.0), (600, 100003, 2000003, 999983, 1.0)])
def test_input_rows_hash_the_previous_token_from_the_step_the_state_slot_or_nothing(dtype, width, buckets, mp, mc, scale):
    from lite_llama_amd.kernels.norm_act import embed_pair
    from oracle import fekanex as O

    torch.manual_seed(width)
    vocab = 50000 if buckets > 1000 else 23
    table, pair = torch.randn(vocab, width).to(dtype), torch.randn(buckets + 1, width).to(dtype)
    seqs = {1: torch.randint(0, vocab, (9,)).tolist(), 2: torch.randint(vocab - 5, vocab, (4,)).tolist(), 0: torch.randint(0, vocab, (6,)).tolist()}
    cfg = {"embedding": {"scale": scale, "bigram": {"buckets": buckets, "mul_prev": mp, "mul_cur": mc}}}
    want = {s: O.embed(t, {"embed": d(table), "bigram": d(pair)}, cfg) for s, t in seqs.items()}
    state = torch.full((2, 4), vocab - 1, dtype=torch.int32, device=DEV)        # stale: a sequence that starts must not read it
    # (slot, first, count): a start, a start of one token, then portions that begin inside the sequences, single tokens
    plan = [[(1, 0, 3), (2, 0, 1)], [(2, 1, 1), (1, 3, 1), (0, 0, 6)], [(1, 4, 5), (2, 2, 2)]]
    parity = {0: 0, 1: 0, 2: 0}
    got = {s: [] for s in seqs}
    for entries in plan:
        step = _step([(s, f, c, parity[s]) for s, f, c in entries])
        toks = torch.tensor([t for s, f, c in entries for t in seqs[s][f:f + c]], dtype=torch.int32, device=DEV)
        x = embed_pair(toks, table.to(DEV), scale, pair.to(DEV), mp, mc, step, state)
        assert x.dtype == torch.float32
        at = 0
        for s, f, c in entries:
            got[s].append(x[at:at + c])
            at += c
            parity[s] ^= 1
    for s in seqs:
        _close(torch.cat(got[s]), want[s], 1e-6)
    # no table: the scaled embedding alone
    x = embed_pair(torch.tensor(seqs[1], dtype=torch.int64, device=DEV), table.to(DEV), scale)
    _close(x, d(table)[seqs[1]] * scale, 1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width,parts,row", [(96, 3, True), (70, 2, True), (2048, 1, False), (4100, 4, True), (64, 0, True)])
def test_residual_norm_adds_a_row_and_part_rows_and_scales_its_output(dtype, width, parts, row):
    from lite_llama_amd.kernels.norm_act import SummedUpdate, add_rmsnorm_shift
    from oracle import fekanex as O

    torch.manual_seed(width + parts)
    n, eps = 6, 1e-5
    x = torch.randn(n, width, device=DEV) * 3
    r = torch.randn(n, width, device=DEV).to(dtype) if row else None
    p = torch.randn(n, parts, width, device=DEV).to(dtype) if parts else None
    w = (1 + 0.1 * torch.randn(width, device=DEV)).to(dtype)
    total = (d(r) if row else 0) + (d(p).sum(1) if parts else 0)
    want_x = d(x) + total
    upd = SummedUpdate(r, p)
    _close(upd.total(), total, 1e-6)
    x1 = x.clone()
    h, res = add_rmsnorm_shift(x1, upd, w, eps, x_out=x1, out_scale=2.5)
    assert res is x1
    _close(x1, want_x, 2e-6)
    _close(h, O.rms_norm(want_x, d(w), eps) * 2.5, TOL[dtype])
    pick = torch.tensor([4, 1], device=DEV)
    x2 = x[pick].contiguous()
    h2, _ = add_rmsnorm_shift(x2, upd.rows(pick), w, eps, x_out=x2)
    _close(x2, want_x[[4, 1]], 2e-6)
    _close(h2, O.rms_norm(want_x[[4, 1]], d(w), eps), TOL[dtype])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("ff,off", [(40, 16), (37, 5)])     # (37: the plain form; 40 behind 16 columns: 16-byte pieces)
def test_clamped_activation_limits_both_sides_and_writes_a_column_range(dtype, ff, off):
    from lite_llama_amd.kernels.norm_act import glu_act

    torch.manual_seed(ff)
    rows = (torch.randn(9, 2 * ff + 3, device=DEV) * 3).to(dtype)
    out = torch.full((9, off + ff + 8), 7.0, device=DEV).to(dtype)
    g, u = d(rows[:, :ff]), d(rows[:, ff:2 * ff])
    for limit in (0.75, 2.0, 100.0):
        gl, ul = torch.clamp(g, max=limit), torch.clamp(u, -limit, limit)
        want = gl * torch.sigmoid(1.702 * gl) * (ul + 1)
        got = glu_act(rows, ff, "clamped", limit=limit, slope=1.702, out=out[:, off:off + ff])
        assert got.data_ptr() == out[:, off:].data_ptr()
        _close(out[:, off:off + ff], want, TOL[dtype])
        assert torch.all(out[:, :off] == 7.0) and torch.all(out[:, off + ff:] == 7.0)
        _close(glu_act(rows, ff, "clamped", limit=limit, slope=1.702), want, TOL[dtype])
    assert (g > 2.0).any() and (u < -2.0).any() and (u > 2.0).any()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("experts,top,width", [(6, 2, 96), (9, 1, 60), (4, 4, 33), (64, 6, 128), (1, 1, 16), (8, 3, 40)])
def test_router_chooses_the_largest_logits_and_weighs_them_by_their_own_softmax(dtype, experts, top, width):
    from lite_llama_amd.kernels.fused_moe import group_router
    from oracle import fekanex as O

    torch.manual_seed(experts * 7 + top)
    n = 37
    h = torch.randn(n, width, device=DEV).to(dtype)
    wr = (torch.randn(experts, width, device=DEV) * 3.0 * width ** -0.5).to(dtype)
    ids, weights, extra = group_router(h, wr, top, scoring="softmax_chosen")
    want_ids, want_w = O.route(d(h), d(wr), top)
    assert extra is None and ids.dtype == torch.int32 and weights.dtype == torch.float32
    logits = d(h) @ d(wr).T
    best = torch.topk(logits, min(top + 1, experts), -1).values
    gap = best.diff(dim=-1).abs().min(-1).values > 1e-4 if best.shape[1] > 1 else torch.ones(n, dtype=torch.bool)   # (no close calls)
    assert gap.sum() > n // 2
    assert torch.equal(ids.cpu().long()[gap], want_ids[gap])
    _close(weights[gap.to(DEV)], want_w[gap], 1e-5)
    assert torch.allclose(weights.sum(-1).cpu(), torch.ones(n), atol=1e-5)


def _conv_case(dtype, heads, kv_heads, dk, dv, taps, pairs, plan, lens, blend, unit_norm=True, bias=True, rot_kw=None):
    """Runs ``conv_rope_cache`` over ``plan`` (steps of ``(slot, first, count)``) and returns per sequence
    ``(queries, cached keys, cached values)`` next to what the oracle's functions give for the whole sequences."""
    from lite_llama_amd.kernels.attention import conv_rope_cache
    from lite_llama_amd.model_layers import RotarySpec
    from oracle import fekanex as O

    torch.manual_seed(dk * 31 + taps)
    channels = (heads + kv_heads) * dk + kv_heads * dv
    eps = 1e-5
    rot = T.rot(2 * pairs, **(rot_kw or {})) if pairs else None
    rows = {s: (torch.randn(n, channels + 5) * 2).to(dtype) for s, n in lens.items()}       # (+ 5: columns of another sublayer)
    b = (torch.randn(channels) * 0.5).to(dtype) if bias else None
    cw = (torch.randn(channels, taps) * 0.6 + 0.3).to(dtype) if taps else None
    lam = torch.tensor([0.375]).to(dtype)
    total_rows = 4 * max(lens.values()) + 16
    table = torch.randperm(total_rows)[:4 * max(lens.values())].view(4, -1).to(torch.int32)
    src = torch.randn(total_rows, kv_heads, dv).to(dtype)
    want = {}
    for s, r in rows.items():
        n = r.shape[0]
        u = d(r[:, :channels]) + (d(b) if bias else 0)
        y = O.causal_conv(u, d(cw)) if taps else u
        q, k = y[:, :heads * dk].view(n, heads, dk), y[:, heads * dk:(heads + kv_heads) * dk].view(n, kv_heads, dk)
        v = y[:, (heads + kv_heads) * dk:].view(n, kv_heads, dv)
        if pairs:
            q, k = O.rotate_pairs(q, torch.arange(n), rot, torch.float32), O.rotate_pairs(k, torch.arange(n), rot, torch.float32)
        if unit_norm:
            q, k = O.rms_norm(q, None, eps), O.rms_norm(k, None, eps)
        if blend:
            v = (1 - d(lam)) * v + d(lam) * d(src)[table[s, :n].long()]
        want[s] = (q, k, v)
    freq = None
    if pairs:
        values, amp = RotarySpec.from_config(rot).table()
        freq = torch.tensor(values, dtype=torch.float64).to(torch.float32).to(DEV)
    else:
        amp = 1.0
    k_cache = torch.full((total_rows, kv_heads, dk), 5.0).to(dtype).to(DEV)
    v_cache = torch.full((total_rows, kv_heads, dv), 5.0).to(dtype).to(DEV)
    state = torch.full((2, 4, max(taps - 1, 1), channels), 9.0).to(dtype).to(DEV) if taps > 1 else None    # stale rows everywhere
    parity = {s: 0 for s in lens}
    got_q = {s: [] for s in lens}
    for entries in plan:
        step = _step([(s, f, c, parity[s]) for s, f, c in entries], table)
        batch = torch.cat([rows[s][f:f + c] for s, f, c in entries]).to(DEV)
        q = conv_rope_cache(batch, heads, kv_heads, dk, dv, step, k_cache, v_cache, bias=b.to(DEV) if bias else None,
                            conv_weight=cw.to(DEV) if taps else None, conv_state=state, freq=freq, pairs=pairs, amp=amp,
                            unit_norm=unit_norm, eps=eps, v_source=src.to(DEV) if blend else None,
                            v_blend=lam.to(DEV) if blend else None)
        at = 0
        for s, f, c in entries:
            got_q[s].append(q[at:at + c])
            at += c
            parity[s] ^= 1
    out = {}
    for s, n in lens.items():
        idx = table[s, :n].long().to(DEV)
        out[s] = (torch.cat(got_q[s]), k_cache[idx], v_cache[idx])
    return out, want


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv_heads,dk,dv,taps,pairs,blend", [(4, 2, 16, 8, 4, 4, True), (3, 1, 12, 10, 3, 3, False),
                                                                   (2, 2, 24, 16, 2, 12, True), (1, 1, 2, 1, 1, 1, True),
                                                                   (2, 1, 136, 200, 5, 20, False), (2, 1, 9, 5, 0, 0, True),
                                                                   (1, 1, 520, 264, 7, 130, True)])
def test_convolution_rotation_unit_norm_and_value_blend_over_portions_of_every_size(dtype, heads, kv_heads, dk, dv, taps, pairs, blend):
    """Portions of one and two tokens right after a sequence's start (fewer tokens behind them than taps), portions longer
    than the taps, single decoded tokens, two sequences side by side, stale rows in every state slot."""
    lens = {1: 23, 3: 9, 0: 4}
    plan = [[(1, 0, 1), (3, 0, 2)], [(1, 1, 1)], [(1, 2, 2), (3, 2, 1), (0, 0, 4)], [(1, 4, 9), (3, 3, 1)], [(3, 4, 5), (1, 13, 1)],
            [(1, 14, 1)], [(1, 15, 8)]]
    got, want = _conv_case(dtype, heads, kv_heads, dk, dv, taps, pairs, plan, lens, blend)
    for s in lens:
        for g, w in zip(got[s], want[s]):
            _close(g, w, 3e-6 if dtype == torch.float32 else TOL[dtype])


def test_convolution_without_bias_norm_or_rotation_is_the_plain_weighted_sum():
    lens = {2: 11}
    got, want = _conv_case(torch.float32, 2, 1, 8, 8, 3, 0, [[(2, 0, 2)], [(2, 2, 1)], [(2, 3, 8)]], lens, False, unit_norm=False, bias=False)
    for g, w in zip(got[2], want[2]):
        _close(g, w, 2e-6)


def test_rotation_far_out_takes_the_angle_in_32_bits():
    """Positions beyond 4000: the product position * frequency is rounded to 32 bits before cos / sin, as the oracle does when
    told to; sequences are placed there through the step's positions."""
    from lite_llama_amd.kernels.attention import conv_rope_cache
    from lite_llama_amd.model_layers import RotarySpec
    from oracle import fekanex as O

    torch.manual_seed(5)
    rot = T.rot(16, base=10000.0, factor=8.0, original=40, fast=8.0, slow=1.0)
    values, amp = RotarySpec.from_config(rot).table()
    freq = torch.tensor(values, dtype=torch.float64).to(torch.float32).to(DEV)
    rows = torch.randn(6, 2 * 16 + 8, device=DEV)
    pos = [4093, 4094, 4095, 4096, 4097, 4098]
    table = torch.zeros(1, 5000, dtype=torch.int32)
    table[0, 4093:4099] = torch.arange(6, dtype=torch.int32)
    step = _step([(0, 4093, 6, 0)], table)
    kc, vc = torch.zeros(8, 1, 16, device=DEV), torch.zeros(8, 1, 8, device=DEV)
    q = conv_rope_cache(rows, 1, 1, 16, 8, step, kc, vc, freq=freq, pairs=8, amp=amp)
    want = O.rotate_pairs(d(rows[:, :16]).view(6, 1, 16), torch.tensor(pos), rot, torch.float32)
    _close(q, want, 2e-6)
    _close(kc[:6], O.rotate_pairs(d(rows[:, 16:32]).view(6, 1, 16), torch.tensor(pos), rot, torch.float32), 2e-6)


def _attention_case(dtype, heads, kv_heads, dk, dv, total, plan, window, keep, hot=None, scale=0.3, sink=True, low=False):
    """Queries against a paged cache through the attention kernels, fed by ``plan`` (steps of ``(slot, first, count)``);
    returns (got, want) of the slot-1 sequence.  ``hot``: one key whose score towers over the rest for every query that may
    see it; ``low``: every score far below 0, so that the sink holds nearly all the weight."""
    from lite_llama_amd.kernels.attention import ragged_attention
    from oracle import fekanex as O

    torch.manual_seed(total + heads + keep)
    group = heads // kv_heads
    q = torch.randn(total, heads, dk)
    k = torch.randn(total, kv_heads, dk)
    v = torch.randn(total, kv_heads, dv)
    if hot is not None:
        u = torch.nn.functional.normalize(torch.randn(dk), dim=0)
        k[hot] = 9.0 * u
        q = q + 9.0 * u
    if low:
        u = torch.nn.functional.normalize(torch.randn(dk), dim=0)
        k, q = k + 8.0 * u, q - 8.0 * u
    q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
    rows_total = 2 * total + 64
    table = torch.randperm(rows_total)[:2 * total].view(2, total).to(torch.int32).to(DEV)
    kc = torch.randn(rows_total, kv_heads, dk).to(dtype).to(DEV)
    vc = torch.randn(rows_total, kv_heads, dv).to(dtype).to(DEV)
    kc[table[1].long()], vc[table[1].long()] = k.to(DEV), v.to(DEV)
    q0 = torch.randn(total, heads, dk).to(dtype)
    zeros = torch.zeros(heads, dtype=dtype, device=DEV) if sink else None
    got = []
    for seqs in plan:
        step = _step([(s, f, c, 0) for s, f, c in seqs], table.cpu())
        qs = torch.cat([(q if s == 1 else q0)[f:f + c] for s, f, c in seqs]).to(DEV).contiguous()
        wide = torch.full((qs.shape[0], heads * dv + 24), 3.0, dtype=dtype, device=DEV)     # the output is a column range of wider rows
        ragged_attention(qs, kc, vc, scale, step, table, sink=zeros, window=window, keep_first=keep, out=wide[:, 8:8 + heads * dv])
        assert torch.all(wide[:, :8] == 3.0) and torch.all(wide[:, 8 + heads * dv:] == 3.0)
        at = 0
        for s, f, c in seqs:
            if s == 1:
                got.append(wide[at:at + c, 8:8 + heads * dv])
            at += c
    mask = O.visible(total, window if window else total + 1, keep)
    outs = []
    for a in range(heads):
        g = a // group
        s = d(q)[:, a] @ d(k)[:, g].T * scale
        if sink:
            w = O.sink_softmax(s, mask)
        else:
            w = torch.softmax(s.masked_fill(~mask, float("-inf")), -1)
        outs.append(w @ d(v)[:, g])
    return torch.cat(got), torch.cat(outs, -1)


SHAPES = [(4, 2, 16, 8), (3, 3, 12, 10), (20, 1, 8, 8), (2, 1, 136, 40)]   # matrix-core form / plain form / two column tiles / wide keys


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", SHAPES[:2])
@pytest.mark.parametrize("keep,hot", [(1, 0), (4, 3), (4, 4), (40, 39), (40, 40), (70, 64), (300, 255), (300, 256), (300, 299), (300, 300)])
def test_kept_first_keys_reach_tokens_far_behind_them_and_the_next_key_does_not(dtype, shape, keep, hot):
    """700 positions in pages of 64, a window of 50: a dominating key at ``hot`` inside the kept first keys decides the output
    of every later token, from prompt portions and from decoded tokens alike; one position further (hot == keep) it is seen
    only while the window still holds it."""
    total, window = 700, 50
    plan = [[(1, 0, 300), (0, 0, 5)], [(1, 300, 2)], [(1, 302, 388)]] + [[(0, 5 + i, 1), (1, 690 + i, 1)] for i in range(10)]
    got, want = _attention_case(dtype, *shape, total, plan, window, keep, hot=hot)
    _close(got, want, 5e-5 if dtype == torch.float32 else 3e-2)
    far = want[hot + window + 5:]
    assert (got[hot + window + 5:].float().cpu() - far).abs().max() < 0.1 * want.abs().max()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("window,keep,hot", [(1, 0, 5), (1, 2, 5), (9, 3, 40), (21, 5, 300), (64, 1, 191), (100, 33, 256), (300, 4, 70),
                                             (6, 11, 20)])
def test_window_edge_with_kept_keys_in_prompts_and_in_decoding(dtype, shape, window, keep, hot):
    """The dominating key sits at ``hot`` (behind the kept keys): position hot + window - 1 still sees it, hot + window does
    not.  The edge is crossed once inside a prompt portion and (in a second run) by decoded tokens; windows shorter and longer
    than a tile, a page and a context partition; more kept keys than the window holds."""
    total = hot + window + 40
    edge = hot + window
    prompt = [[(1, 0, 7), (0, 0, 3)], [(1, 7, total - 7)]]
    decode = [[(1, 0, edge - 3)]] + [[(1, i, 1), (0, i - edge + 3, 1)] for i in range(edge - 3, total)]
    for plan in (prompt, decode):
        got, want = _attention_case(dtype, *shape, total, plan, window, keep, hot=hot)
        _close(got, want, 5e-5 if dtype == torch.float32 else 3e-2)
        gap = (want[edge - 1] - want[edge]).abs().max()              # the outputs on the two sides of the edge differ grossly
        assert gap > 0.5 and (got[edge - 1:edge + 1].float().cpu() - want[edge - 1:edge + 1]).abs().max() < 0.05 * gap


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", SHAPES[:3])
def test_sink_of_score_zero_takes_the_weight_when_every_score_is_low(dtype, shape):
    """Scores around -20: without the sink the output is an average of values, with it nearly nothing; and with ordinary
    scores the sink's 1 in the denominator still shows."""
    total = 300
    plan = [[(1, 0, 280)]] + [[(1, 280 + i, 1)] for i in range(20)]
    got, want = _attention_case(dtype, *shape, total, plan, 30, 2, low=True)
    assert want.abs().max() < 0.02 and (got.float().cpu() - want).abs().max() < 1e-3
    plain, _ = _attention_case(dtype, *shape, total, plan, 30, 2, low=True, sink=False)
    assert plain.float().abs().max() > 0.5
    got, want = _attention_case(dtype, *shape, total, plan, 30, 2, scale=0.1)
    _close(got, want, 5e-5 if dtype == torch.float32 else 3e-2)
    none, _ = _attention_case(dtype, *shape, total, plan, 30, 2, scale=0.1, sink=False)
    assert (none.float().cpu() - want).abs().max() > 0.02


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_first_tokens_of_a_sequence_see_exactly_themselves(dtype):
    """Positions 0 .. 3 with a window of 2 and 3 kept keys, token by token and as one portion."""
    for plan in ([[(1, 0, 6)]], [[(1, i, 1)] for i in range(6)], [[(1, 0, 2)], [(1, 2, 4)]]):
        got, want = _attention_case(dtype, 4, 2, 16, 8, 6, plan, 2, 3)
        _close(got, want, 5e-5 if dtype == torch.float32 else 3e-2)


# ------------------------------------------------------------------------------------------------------------------- #
# whole models: loader -> runner -> cache
# ------------------------------------------------------------------------------------------------------------------- #
_MODELS = {}


def _model(tmp_path_factory, name, dtype):
    from lite_llama_amd.weights import load_pretrained

    key = (name, dtype)
    if key not in _MODELS:
        cfg = T.CONFIGS[name]
        tens = T.tensors(cfg, seed=len(name))
        folder = L.write(tmp_path_factory.mktemp(name), cfg, tens)
        _MODELS[key] = (load_pretrained(folder, device=DEV, dtype=dtype), cfg, tens, folder)
    return _MODELS[key]


@pytest.mark.parametrize("name", sorted(T.CONFIGS))
def test_whole_prompt_layers_and_logits(tmp_path_factory, name):
    from lite_llama_amd.executor.ragged import RaggedRunner
    from oracle import fekanex as O

    model, cfg, tens, _ = _model(tmp_path_factory, name, torch.float32)
    toks = L.prompt(cfg, 45)
    layers = []
    want = O.forward(toks, tens, cfg, layers_out=layers)
    runner = RaggedRunner(model, 64, 2, block_size=16, device=DEV)
    got_layers = []
    got = runner.step([(runner.admit(), toks)], list(range(len(toks))), collect_layers=got_layers)
    runner.check_errors()
    assert len(got_layers) == len(layers)
    for g, w in zip(got_layers, layers):
        _close(g, w, 2e-5)
    _close(got, want, 2e-5)


@pytest.mark.parametrize("name", sorted(T.CONFIGS))
@pytest.mark.parametrize("sizes", [[1], [2], [3, 2, 7, 1, 16, 5], [40, 1]])
def test_portions_and_token_by_token_decoding_equal_the_whole_prompt(tmp_path_factory, name, sizes):
    """Portions down to two tokens, pure token-by-token decoding from the first token on, and a long portion followed by
    decoding; pages of 8 tokens, so portions, windows, taps and pages start and end inside one another."""
    from lite_llama_amd.executor.ragged import RaggedRunner
    from oracle import fekanex as O

    model, cfg, tens, _ = _model(tmp_path_factory, name, torch.float32)
    toks = L.prompt(cfg, 58, seed=1)
    want = O.forward(toks, tens, cfg)
    runner = RaggedRunner(model, 64, 2, block_size=8, device=DEV)
    _close(_feed(runner, runner.admit(), toks, sizes), want, 2e-5)
    runner.check_errors()


@pytest.mark.parametrize("name", ["mix", "odd"])
def test_unequal_requests_in_one_batch_equal_each_alone_and_freed_pages_and_slots_are_used_again(tmp_path_factory, name):
    """Four requests of different lengths ride together in changing portions, three slots and a pool that only holds them
    because finished requests give their pages back; a late request takes over a used slot (with the carried rows and the
    previous token its last owner left) and used pages."""
    from lite_llama_amd.executor.ragged import RaggedRunner
    from oracle import fekanex as O

    model, cfg, tens, _ = _model(tmp_path_factory, name, torch.float32)
    lens = {"a": 41, "b": 9, "c": 26, "d": 33}
    toks = {k: L.prompt(cfg, n, seed=ord(k)) for k, n in lens.items()}
    want = {k: O.forward(v, tens, cfg) for k, v in toks.items()}
    runner = RaggedRunner(model, 96, 3, block_size=8, device=DEV)      # 12 pages: a + b + c need 11, d needs 5
    sizes = {"a": [5, 1, 1, 9, 2, 30], "b": [2, 1, 3, 1, 1, 1], "c": [1, 13, 2, 2, 8], "d": [16, 1, 1, 15]}
    at, slot, got, k = {x: 0 for x in lens}, {}, {x: [] for x in lens}, 0
    waiting, live = ["a", "b", "c", "d"], []
    while waiting or live:
        while waiting and runner.free_slots and runner.blocks_held() + runner.blocks_for(lens[waiting[0]]) <= runner.total_blocks:
            who = waiting.pop(0)
            slot[who] = runner.admit()
            live.append(who)
        entries, rows, owners, base = [], [], [], 0
        for who in live:
            if (k + ord(who)) % 4 == 0 and len(live) > 1:
                continue                                              # left out of this step, goes on later
            c = min(sizes[who][min(k, len(sizes[who]) - 1)], lens[who] - at[who])
            entries.append((slot[who], toks[who][at[who]:at[who] + c]))
            rows += range(base, base + c)
            owners += [who] * c
            base, at[who] = base + c, at[who] + c
        k += 1
        if not entries:
            continue
        out = runner.step(entries, rows)
        for j, who in enumerate(owners):
            got[who].append(out[j:j + 1])
        ended = [n for n in live if at[n] == lens[n]]
        runner.release([slot[n] for n in ended])
        live = [n for n in live if n not in ended]
    runner.check_errors()
    assert slot["d"] in (slot["a"], slot["b"], slot["c"])
    assert runner.cache.free_blocks == runner.total_blocks
    for who in lens:
        _close(torch.cat(got[who]), want[who], 2e-5)


@pytest.mark.parametrize("name", ["odd", "wide"])
def test_long_decoding_past_windows_and_over_many_pages(tmp_path_factory, name):
    from lite_llama_amd.executor.ragged import RaggedRunner
    from oracle import fekanex as O

    model, cfg, tens, _ = _model(tmp_path_factory, name, torch.float32)
    toks = L.prompt(cfg, 150, seed=5)
    want = O.forward(toks, tens, cfg)
    runner = RaggedRunner(model, 160, 1, block_size=16, device=DEV)
    _close(_feed(runner, runner.admit(), toks, [6, 1]), want, 3e-5)


@pytest.mark.parametrize("name", sorted(T.CONFIGS))
def test_bfloat16_model_tracks_the_oracle_and_its_own_portions(tmp_path_factory, name):
    from lite_llama_amd.executor.ragged import RaggedRunner
    from oracle import fekanex as O

    model, cfg, tens, _ = _model(tmp_path_factory, name, torch.bfloat16)
    toks = L.prompt(cfg, 70, seed=2)
    want = O.forward(toks, tens, cfg)
    runner = RaggedRunner(model, 160, 2, block_size=16, device=DEV)
    whole = _feed(runner, runner.admit(), toks, [70]).float().cpu()
    parts = _feed(runner, runner.admit(), toks, [2, 9, 1, 1, 30, 1]).float().cpu()
    spread = want.std().item()
    # medians over the tokens: a token whose router sees two experts within a rounding step of each other may choose the other
    err = lambda a, b: (a.to(F64) - b.to(F64)).pow(2).mean(-1).sqrt().median().item()   # noqa: E731
    assert err(whole, want) < 0.06 * spread
    assert err(parts, whole) < 0.04 * spread


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_captured_decode_steps_replay_like_eager_ones(tmp_path_factory, dtype):
    from lite_llama_amd.executor.ragged import RaggedRunner

    model, cfg, _, _ = _model(tmp_path_factory, "mix", dtype)
    a, b = L.prompt(cfg, 290, seed=21), L.prompt(cfg, 40, seed=22)
    eager = RaggedRunner(model, 512, 2, block_size=16, device=DEV)
    graph = RaggedRunner(model, 512, 2, block_size=16, device=DEV, capture_decode=True)
    out = {"eager": [], "graph": []}
    for name, r in (("eager", eager), ("graph", graph)):
        sa, sb = r.admit(), r.admit()
        r.step([(sa, a[:240])], [])
        for i in range(240, 262):                                   # one sequence decoding across a partition edge
            out[name].append(r.step([(sa, a[i:i + 1])]).float().cpu().clone())
        r.step([(sa, a[262:263]), (sb, b[:30])], [])
        for i in range(10):                                         # two sequences decoding together
            out[name].append(r.step([(sa, a[263 + i:264 + i]), (sb, b[30 + i:31 + i])]).float().cpu().clone())
        r.release([sb])
        for i in range(273, 290):
            out[name].append(r.step([(sa, a[i:i + 1])]).float().cpu().clone())
        r.check_errors()
    assert graph.replays >= 40 and eager.replays == 0
    for e, g2 in zip(out["eager"], out["graph"]):
        assert torch.allclose(e, g2, rtol=0, atol=1e-6 if dtype == torch.float32 else 2e-2), (e - g2).abs().max()


# ------------------------------------------------------------------------------------------------------------------- #
# entry points: engine, command line, trace replay
# ------------------------------------------------------------------------------------------------------------------- #
def test_engine_generates_greedily_like_the_oracle(tmp_path_factory):
    from lite_llama_amd.engine import GenerationEngine, SamplingParams
    from oracle import fekanex as O

    model, cfg, tens, _ = _model(tmp_path_factory, "odd", torch.float32)
    prompts = [L.prompt(cfg, n, seed=n) for n in (3, 19, 1, 11, 7)]
    engine = GenerationEngine(model, max_tokens=96, max_requests=3, block_size=8, max_step_tokens=10, device=DEV)
    outs = engine.generate(prompts, SamplingParams(max_new_tokens=6))
    for p, o in zip(prompts, outs):
        assert o == O.greedy(p, tens, cfg, 6)
    captured = GenerationEngine(model, max_tokens=96, max_requests=3, block_size=8, max_step_tokens=10, device=DEV, capture_decode=True)
    assert captured.generate(prompts, SamplingParams(max_new_tokens=6)) == outs and captured.runner.replays > 0
    assert engine.runner.cache.free_blocks == engine.runner.total_blocks and engine.runner.free_slots == 3
    sampled = engine.generate(prompts[:2], SamplingParams(max_new_tokens=5, temperature=0.8, top_p=0.9, repetition_penalty=1.2))
    assert [len(s) for s in sampled] == [5, 5] and all(0 <= t < cfg["vocab"] for s in sampled for t in s)
    with pytest.raises(ValueError):
        engine.runner.step([(engine.runner.admit(), [cfg["vocab"]])])


def test_command_line_generate_and_trace_replay(tmp_path_factory, tmp_path):
    from oracle import fekanex as O

    _, cfg, tens, folder = _model(tmp_path_factory, "wide", torch.float32)
    prompt = L.prompt(cfg, 9, seed=4)
    env = dict(os.environ, PYTHONPATH=ROOT)
    done = subprocess.run([sys.executable, "-m", "lite_llama_amd", "generate", "--model", folder, "--dtype", "float32",
                           "--prompt-ids", ",".join(map(str, prompt)), "--max-new-tokens", "4"],
                          capture_output=True, text=True, env=env, cwd=ROOT, timeout=300)
    assert done.returncode == 0, done.stderr[-2000:]
    line = json.loads(done.stdout.strip().splitlines()[-1])
    assert line["prompt"] == prompt and line["generated"] == O.greedy(prompt, tens, cfg, 4)

    a, b = L.prompt(cfg, 31, seed=8), L.prompt(cfg, 6, seed=9)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:13], "want": [0, 12]}, {"id": "b", "tokens": b[:2], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "b", "tokens": b[2:], "want": [3]}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": a[13:30], "want": []}], "end": []},
             {"step": 3, "entries": [{"id": "a", "tokens": a[30:], "want": [0]}, {"id": "c", "tokens": b, "want": [5]}], "end": ["a", "c"]}]
    out = tmp_path / "out"
    done = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32", "--out", str(out),
                           "--max-tokens", "128"], input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True,
                          text=True, env=env, cwd=ROOT, timeout=300)
    assert done.returncode == 0, done.stderr[-2000:]
    assert [ln for ln in done.stdout.splitlines() if ln.startswith("done")] == [f"done {i}" for i in range(4)]
    import numpy as np

    la, lb = O.forward(a, tens, cfg), O.forward(b, tens, cfg)
    read = lambda i: torch.from_numpy(np.fromfile(out / f"{i}.f32", dtype="<f4")).view(-1, cfg["vocab"])   # noqa: E731
    _close(read(0), la[[0, 12]], 2e-5)
    _close(read(1), lb[[5]], 2e-5)
    assert not (out / "2.f32").exists()
    _close(read(3), torch.stack([la[30], lb[5]]), 2e-5)


def _random_config(seed):
    """A configuration drawn from the whole range the reader takes: head counts and widths with and without the matrix-core
    forms' multiples, 1 - 6 taps or none, windows from 1 key to longer than the prompt, kept keys from none to more than the
    window, rotations of a part or all of a head with and without scaling, every feed-forward kind in any order, blending
    layers anywhere."""
    import random

    r = random.Random(seed)
    kv = r.choice([1, 2, 3])
    dv = r.choice([8, 16, 24, 10, 48])
    layers = []
    for _ in range(r.randint(1, 4)):
        mixes = r.random() < 0.7
        g = kv if mixes else r.choice([1, 2])
        heads = g * r.choice([1, 2, 4, 5])
        dim = r.choice([8, 16, 32, 64, 12, 20, 128])
        vdim = dv if mixes else r.choice([8, 12, 32])
        dims = r.choice([dim, dim // 2, 2, max(2, (dim // 4) * 2)])
        kind = r.choice(["dense", "moe", None])
        experts = r.randint(1, 9)
        mlp = T.dense(r.choice([16, 40, 44]), limit=r.choice([0.5, 2.0, 30.0])) if kind == "dense" else \
            T.moe(experts, r.randint(1, experts), r.choice([8, 12, 24])) if kind == "moe" else None
        layers.append(T.attention(heads, g, dim, vdim, r.choice([None, 1, 2, 3, 4, 6]), r.choice([1, 3, 8, 17, 40, 64, 200]),
                                  r.choice([0, 0, 1, 2, 5, 33, 70]), dims, v_mix=mixes, mlp=mlp, scaled=r.random() < 0.7,
                                  base=r.choice([100.0, 10000.0]), factor=r.choice([2.0, 4.0, 16.0]), original=r.choice([16, 64, 1024]),
                                  scale=r.choice([0.5, 1.0, 2.0]) * dim ** -0.5 * 4))
    return T.config(layers, width=r.choice([32, 48, 60, 88]), vocab=r.randint(20, 300), buckets=r.randint(1, 500),
                    mul_prev=r.randint(0, 1000), mul_cur=r.randint(1, 1000), scale=r.choice([1.0, 0.25, 3.0]),
                    logit_scale=r.choice([1.0, 0.125, 5.0]), eps=r.choice([1e-5, 1e-6, 1e-3]))


@pytest.mark.parametrize("seed", range(12))
def test_random_configurations_whole_in_portions_decoded_and_side_by_side(tmp_path, seed):
    from lite_llama_amd.executor.ragged import RaggedRunner
    from lite_llama_amd.weights import load_pretrained
    from oracle import fekanex as O

    cfg = _random_config(seed)
    tens = T.tensors(cfg, seed=seed)
    model = load_pretrained(L.write(tmp_path / "m", cfg, tens), device=DEV, dtype=torch.float32)
    a, b = L.prompt(cfg, 90, seed=seed), L.prompt(cfg, 37, seed=seed + 50)
    wa, wb = O.forward(a, tens, cfg), O.forward(b, tens, cfg)
    runner = RaggedRunner(model, 256, 3, block_size=16, device=DEV)
    _close(_feed(runner, runner.admit(), a, [90]), wa, 3e-5)
    _close(_feed(runner, runner.admit(), a, [2, 1, 7, 3, 1, 30, 1]), wa, 3e-5)
    runner.release([0, 1])
    sa, sb = runner.admit(), runner.admit()            # used slots and pages again, two requests side by side
    got_a, got_b, ia, ib = [], [], 0, 0
    for ca, cb in [(11, 1), (1, 2), (40, 1), (1, 20), (5, 1), (32, 12)]:
        out = runner.step([(sa, a[ia:ia + ca]), (sb, b[ib:ib + cb])], list(range(ca + cb)))
        got_a.append(out[:ca])
        got_b.append(out[ca:])
        ia, ib = ia + ca, ib + cb
    assert ia == 90 and ib == 37
    runner.check_errors()
    _close(torch.cat(got_a), wa, 3e-5)
    _close(torch.cat(got_b), wb, 3e-5)
