"""Nivotar on the GPU against the plain CPU restatement (oracle/nivotar.py): each mechanism's kernels alone, then whole models
built from small random checkpoints through the loader, the ragged runner, the paged state cache, the generation engine and
the command line.  float32 runs are held to rounding error; bfloat16 runs to the rounding of their activations.  Where random
weights would hide a fault (a key at a window's edge, a value written far back into a slowly decaying state, an identity
expert), inputs are made so that it shows."""

import json
import os
import subprocess
import sys

import pytest
import torch

from tests import _layered as L
from tests import _nivotar as T
from tests.test_layered_gpu import _close, _feed, _step

pytestmark = pytest.mark.gpu
DEV = "cuda"
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
F64 = torch.float64
TOL = {torch.float32: 2e-5, torch.bfloat16: 2e-2}
_MODELS = {}


def d(t):
    return t.detach().cpu().to(F64)


def bf(t):
    """Values a 16-bit tensor holds exactly."""
    return t.to(torch.bfloat16).float()


# ------------------------------------------------------------------------------------------------------------------- #
# mechanisms alone
# ------------------------------------------------------------------------------------------------------------------- #
PLAN = [[(2, 0, 5)], [(2, 5, 1), (0, 0, 2)], [(0, 2, 1), (2, 6, 21), (3, 0, 40)], [(3, 40, 1), (0, 3, 2), (2, 27, 1)], [(3, 41, 18)]]
LENS = {2: 28, 0: 5, 3: 59}


def _walk(plan, lens, dtype, make_rows, run, slots=4, stale=None):
    """Feeds per-sequence rows through ``run(rows of the step, step)`` along a plan of steps ``[(slot, first, count)]`` with the
    parity flipping as the runner flips it; returns ``{slot: [T, ...] outputs}``."""
    full = {s: make_rows(s, n) for s, n in lens.items()}
    parity = {s: 0 for s in lens}
    out = {s: [] for s in lens}
    for seqs in plan:
        rows = torch.cat([full[s][f:f + c] for s, f, c in seqs]).to(DEV).to(dtype)
        got = run(rows, _step([(s, f, c, parity[s]) for s, f, c in seqs], stale))
        at = 0
        for s, f, c in seqs:
            out[s].append(got[at:at + c])
            at += c
            parity[s] ^= 1
    return full, {s: torch.cat(v) for s, v in out.items()}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("kind,heads,qk_heads,dk,dv", [("fixed", 2, 2, 16, 24), ("fixed", 3, 3, 10, 6), ("entry", 3, 3, 16, 8),
                                                     ("entry", 2, 2, 64, 16), ("token", 4, 2, 16, 8), ("token", 3, 3, 6, 10),
                                                     ("token", 4, 2, 128, 32), ("entry", 1, 1, 1, 1), ("fixed", 1, 1, 200, 20)])
def test_decaying_state_over_portions_of_every_size_and_stale_slots(dtype, kind, heads, qk_heads, dk, dv):
    """All three decays of the scan kernel: starts of sequences, single decoded tokens and portions inside a sequence side by
    side; slots hold another owner's state when a sequence starts in them."""
    from lite_llama_amd.kernels.recurrent import linear_scan
    from oracle import nivotar as O

    g = torch.Generator().manual_seed(dk * 7 + dv)
    qk, vw = qk_heads * dk, heads * dv
    extra = heads * dk if kind == "entry" else heads if kind == "token" else 0
    cols = 2 * qk + vw + extra
    state = torch.randn(4, heads, dk, dv, device=DEV)
    decay = bf(torch.rand(heads, generator=g) * 0.5 + 0.5)
    bias = bf(torch.randn(heads * dk, generator=g))
    dt_bias, a_log, skip = bf(torch.randn(heads, generator=g)), bf(torch.rand(heads, generator=g) * 2 - 1.5), bf(torch.randn(heads, generator=g))
    tau = 4.0

    def run(rows, step):
        q, k, v, e = rows[:, :qk], rows[:, qk:2 * qk], rows[:, 2 * qk:2 * qk + vw], rows[:, 2 * qk + vw:]
        if kind == "fixed":
            return linear_scan(q, k, v, heads, dk, dv, step, state, act=True, head_decay=decay.to(DEV))
        if kind == "entry":
            return linear_scan(q, k, v, heads, dk, dv, step, state, q_scale=dk ** -0.5, gate=e, gate_bias=bias.to(DEV).to(dtype), tau=tau)
        return linear_scan(q, k, v, heads, dk, dv, step, state, qk_heads=qk_heads, dt=e, dt_bias=dt_bias.to(DEV).to(dtype),
                           a_log=a_log.to(DEV).to(dtype), skip=skip.to(DEV).to(dtype))

    full, got = _walk(PLAN, LENS, dtype, lambda s, n: bf(torch.randn(n, cols, generator=g) * 0.7), run)
    for s, rows in full.items():
        r = rows.to(F64)
        q, k = r[:, :qk].view(-1, qk_heads, dk), r[:, qk:2 * qk].view(-1, qk_heads, dk)
        v, e = r[:, 2 * qk:2 * qk + vw].view(-1, heads, dv), r[:, 2 * qk + vw:]
        want = torch.zeros(r.shape[0], heads, dv, dtype=F64)
        for h in range(heads):
            j = h // (heads // qk_heads)
            if kind == "fixed":
                want[:, h], _ = O.decay_scan(O.silu(q[:, j]), O.silu(k[:, j]), O.silu(v[:, h]), float(decay[h]))
            elif kind == "entry":
                a = torch.exp(torch.nn.functional.logsigmoid(e.view(-1, heads, dk)[:, h] + bias.to(F64).view(heads, dk)[h]) / tau)
                want[:, h], _ = O.decay_scan(q[:, j] * dk ** -0.5, k[:, j], v[:, h], a)
            else:
                step_size = O.softplus(e[:, h] + float(dt_bias[h]))[:, None]
                o, _ = O.decay_scan(q[:, j], k[:, j], step_size * v[:, h], torch.exp(-torch.exp(a_log[h].to(F64)) * step_size))
                want[:, h] = o + float(skip[h]) * v[:, h]
        _close(got[s], want.view(-1, vw), 3e-5 if dtype == torch.float32 else 2e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_decays_evaluated_ahead_of_the_scan_are_the_ones_evaluated_inside_it(dtype):
    """Runs of several tokens evaluate the per-entry decays in a pass of their own, decoded tokens inside the scan: the same
    bits, so a prompt in one portion and token by token leaves the same state."""
    from lite_llama_amd.kernels.recurrent import linear_scan

    g = torch.Generator().manual_seed(11)
    heads, dk, dv, n = 2, 24, 40, 37
    rows = bf(torch.randn(n, 3 * heads * dk + heads * dv, generator=g) * 2).to(DEV).to(dtype)
    bias = bf(torch.randn(heads * dk, generator=g)).to(DEV).to(dtype)
    qk = heads * dk
    outs, states = [], []
    for plan in ([[(0, 0, n)]], [[(0, p, 1)] for p in range(n)]):
        state = torch.randn(1, heads, dk, dv, device=DEV)
        run = lambda r, step: linear_scan(r[:, :qk], r[:, qk:2 * qk], r[:, 2 * qk:2 * qk + heads * dv], heads, dk, dv, step, state,  # noqa: E731
                                          gate=r[:, 2 * qk + heads * dv:], gate_bias=bias, tau=3.0)
        _, got = _walk(plan, {0: n}, dtype, lambda s, m: rows.cpu().float(), run)
        outs.append(got[0])
        states.append(state.clone())
    assert torch.equal(outs[0], outs[1]) and torch.equal(states[0], states[1])


@pytest.mark.parametrize("decay,far", [(1.0, 0), (0.998, 3), (0.998, 15), (0.998, 16), (0.99, 255)])
def test_a_value_written_far_back_is_read_hundreds_of_tokens_later_through_many_portions(decay, far):
    """One key / value pair at position ``far`` is made large; a query that matches its key reads it 600 tokens later, scaled by
    decay^distance, through portions that end on and off the kernel's token tiles and through decoded tokens."""
    from lite_llama_amd.kernels.recurrent import linear_scan
    from oracle import nivotar as O

    g = torch.Generator().manual_seed(far)
    T_, dk, dv = 700, 16, 8
    rows = bf(torch.randn(T_, 2 * dk + dv, generator=g) * 0.05)
    rows[far, dk:2 * dk] = 0.0
    rows[far, dk + 3] = 4.0
    rows[far, 2 * dk:] = bf(torch.linspace(-8, 8, dv))
    for probe in (600 + far // 4, 699):
        rows[probe, :dk] = 0.0
        rows[probe, 3] = 2.0
    state = torch.randn(2, 1, dk, dv, device=DEV)
    dec = torch.tensor([decay], dtype=torch.float32, device=DEV)
    plan = [[(1, 0, 1)], [(1, 1, 16)], [(1, 17, 47)], [(1, 64, 2)], [(1, 66, 1)], [(1, 67, 500)], [(1, 567, 100)]] \
        + [[(1, p, 1)] for p in range(667, 700)]
    run = lambda r, step: linear_scan(r[:, :dk], r[:, dk:2 * dk], r[:, 2 * dk:], 1, dk, dv, step, state, head_decay=dec)  # noqa: E731
    _, got = _walk(plan, {1: T_}, torch.float32, lambda s, n: rows, run, slots=2)
    r = rows.to(F64)
    want, _ = O.decay_scan(r[:, :dk], r[:, dk:2 * dk], r[:, 2 * dk:], float(dec[0]))
    assert want[699].abs().max() > 5 * want[650].abs().max()          # (the probe reads the far pair, nothing else is as large)
    _close(got[1], want, 3e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("channels,taps", [(40, 3), (37, 1), (24, 2), (300, 6), (8, 4)])
def test_convolution_carries_rows_through_portions_shorter_than_its_taps(dtype, channels, taps):
    from lite_llama_amd.kernels.recurrent import conv_act
    from oracle import nivotar as O

    g = torch.Generator().manual_seed(channels + taps)
    w, b = bf(torch.randn(channels, taps, generator=g) * 0.5), bf(torch.randn(channels, generator=g) * 0.3)
    state = torch.randn(2, 4, max(taps - 1, 1), channels, device=DEV).to(dtype) if taps > 1 else None
    pad = 5                                                            # (the rows are a column range of wider rows)
    run = lambda r, step: conv_act(torch.cat([r.new_zeros(r.shape[0], pad), r], 1)[:, pad:], w.to(DEV).to(dtype),  # noqa: E731
                                   b.to(DEV).to(dtype), step, state)
    full, got = _walk(PLAN, LENS, dtype, lambda s, n: bf(torch.randn(n, channels, generator=g)), run)
    for s, rows in full.items():
        _close(got[s], O.silu(O.causal_conv(rows.to(F64), w.to(F64), b.to(F64))), 3e-6 if dtype == torch.float32 else 2e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width,parts,w_len,gate,first", [(48, 2, 48, "silu", True), (30, 3, 30, "silu", True), (40, 5, 8, "silu", False),
                                                         (128, 1, 128, "sigmoid", False), (600, 1, 600, "sigmoid", False),
                                                         (1, 1, 1, "silu", True), (36, 4, 9, None, False)])
def test_read_out_norm_in_parts_with_the_gate_before_or_after(dtype, width, parts, w_len, gate, first):
    from lite_llama_amd.kernels.recurrent import gated_out_norm
    from oracle import nivotar as O

    torch.manual_seed(width)
    n, eps, scale = 7, 1e-5, 1.3
    o = torch.randn(n, width, device=DEV) * 3
    w = bf(1 + 0.2 * torch.randn(w_len)).to(DEV).to(dtype)
    wide = bf(torch.randn(n, width + 6)).to(DEV).to(dtype)
    out = torch.zeros(n, width + 3, device=DEV, dtype=dtype)
    gated_out_norm(o, w, eps, parts=parts, gate=wide[:, 6:] if gate else None, gate_kind=gate, gate_first=first, scale=scale,
                   out=out[:, 3:])
    gv = d(wide[:, 6:])
    gv = O.silu(gv) if gate == "silu" else torch.sigmoid(gv) if gate == "sigmoid" else torch.ones_like(gv)
    y = d(o) * gv if first else d(o)
    y = O.rms_norm(y.view(n, parts, width // parts), None, eps).view(n, width) * d(w).repeat(width // w_len)
    y = y if first else y * gv
    _close(out[:, 3:], y * scale, 3e-6 if dtype == torch.float32 else 1e-2)
    assert out[:, :3].abs().max() == 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv_heads,dk,dv,dims", [(4, 2, 16, 8, 8), (5, 5, 12, 10, 6), (3, 1, 12, 10, 12), (1, 1, 2, 1, 2),
                                                      (8, 4, 64, 96, 32), (2, 1, 8, 8, 0)])
def test_whole_row_norms_and_half_split_rotation_at_positions_far_out(dtype, heads, kv_heads, dk, dv, dims):
    from lite_llama_amd.kernels.attention import rownorm_rope_cache
    from oracle import nivotar as O

    torch.manual_seed(dk)
    pos = [0, 1, 2, 63, 64, 1000, 4099]
    n, base, eps, vs = len(pos), 50000.0, 1e-5, 0.8
    qn, kn, vn = heads * dk, kv_heads * dk, kv_heads * dv
    rows = bf(torch.randn(n, qn + kn + vn + 3)).to(DEV).to(dtype)
    qw, kw = bf(1 + 0.3 * torch.randn(qn)), bf(1 + 0.3 * torch.randn(kn))
    k_cache, v_cache = torch.zeros(20, kv_heads, dk, device=DEV, dtype=dtype), torch.zeros(20, kv_heads, dv, device=DEV, dtype=dtype)
    select = [3, 17, 0, 9, 5, 12, 1]
    step = _step([(0, 0, 3, 0), (1, 63, 2, 0), (2, 1000, 1, 0), (3, 4099, 1, 0)])
    step.select = torch.tensor(select, dtype=torch.int32, device=DEV)
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F64).to(torch.float32).to(DEV) if dims else None
    q = rownorm_rope_cache(rows, heads, kv_heads, dk, dv, step, k_cache, v_cache, q_weight=qw.to(DEV).to(dtype),
                           k_weight=kw.to(DEV).to(dtype), eps=eps, freq=freq, pairs=dims // 2, value_scale=vs)
    r = d(rows)
    p = torch.tensor(pos)
    want_q = O.rms_norm(r[:, :qn], qw.to(F64), eps).view(n, heads, dk)
    want_k = O.rms_norm(r[:, qn:qn + kn], kw.to(F64), eps).view(n, kv_heads, dk)
    if dims:
        want_q, want_k = O.rotate_half(want_q, p, dims, base), O.rotate_half(want_k, p, dims, base)
    # the angle is a 32-bit product: at position 4099 it is known to 4099 * 2^-24, which is what the rotation's entries may differ by
    tol = 6e-4 if dtype == torch.float32 else 2e-2
    _close(q, want_q, tol)
    _close(k_cache[select], want_k, tol)
    _close(v_cache[select], r[:, qn + kn:qn + kn + vn].view(n, kv_heads, dv) * vs, 1e-6 if dtype == torch.float32 else 1e-2)
    _close(q[:3], want_q[:3], 3e-6 if dtype == torch.float32 else 2e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv_heads,dk,dv", [(4, 2, 16, 8), (3, 1, 12, 10), (20, 1, 8, 8)])
@pytest.mark.parametrize("window,hot", [(1, 5), (9, 40), (21, 300), (64, 191), (80, 63), (100, 256), (300, 70)])
def test_window_edge_in_prompts_and_in_decoding(dtype, heads, kv_heads, dk, dv, window, hot):
    """One key is made to dominate every softmax it takes part in.  The last query that still sees it and the first that does
    not differ grossly; both lie inside a prompt portion in one plan and are decoded tokens in the other; pages of 16."""
    from lite_llama_amd.kernels.attention import ragged_attention, rownorm_rope_cache
    from oracle import nivotar as O

    g = torch.Generator().manual_seed(window * 1000 + hot)
    total, block = hot + window + 7, 16
    qn, kn, vn = heads * dk, kv_heads * dk, kv_heads * dv
    rows = bf(torch.randn(total, qn + kn + vn, generator=g) * 0.3)
    rows[:, :qn] = 1.0                                                  # every query points along the all-ones direction
    rows[hot, qn:qn + kn] = 3.0                                         # ... and so does one key, three times as long
    rows[hot, qn + kn:] = 5.0
    scale = 8.0 / dk
    edge = hot + window - 1                                             # the last position that sees the hot key
    plans = {"prompt": [[(0, 0, hot + 1)], [(0, hot + 1, total - hot - 1)]] if window > 2 else [[(0, 0, total)]],
             "decoded": [[(0, 0, max(edge - 1, 1))]] + [[(0, p, 1)] for p in range(max(edge - 1, 1), total)]}
    pages = -(-total // block)
    table = torch.zeros(1, pages * block, dtype=torch.int32)
    order = torch.randperm(pages, generator=g)
    for p in range(pages * block):
        table[0, p] = int(order[p // block]) * block + p % block
    r = rows.to(F64)
    mask = O.visible(total, window)
    want = []
    for h in range(heads):
        j = h // (heads // kv_heads)
        s = (r[:, h * dk:(h + 1) * dk] @ r[:, qn + j * dk:qn + (j + 1) * dk].T * scale).masked_fill(~mask, -float("inf"))
        want.append(torch.softmax(s, -1) @ r[:, qn + kn + j * dv:qn + kn + (j + 1) * dv])
    want = torch.cat(want, 1)
    assert (want[edge] - want[edge + 1]).abs().max() > 2.0
    for name, plan in plans.items():
        k_cache = torch.randn(pages * block, kv_heads, dk, device=DEV).to(dtype)      # (used pages: stale rows everywhere)
        v_cache = torch.randn(pages * block, kv_heads, dv, device=DEV).to(dtype)

        def run(rws, step):
            q = rownorm_rope_cache(rws, heads, kv_heads, dk, dv, step, k_cache, v_cache)
            return ragged_attention(q, k_cache, v_cache, scale, step, table.to(DEV), window=window)

        _, got = _walk(plan, {0: total}, dtype, lambda s, n: rows, run, stale=table)
        _close(got[0], want, 3e-5 if dtype == torch.float32 else 3e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("experts,identity,top,width", [(6, 2, 3, 96), (5, 0, 1, 60), (3, 2, 5, 33), (10, 3, 4, 128), (1, 1, 1, 16),
                                                       (1, 0, 1, 18), (60, 4, 6, 40)])
def test_router_chooses_by_corrected_score_and_weighs_by_the_score_alone(dtype, experts, identity, top, width):
    from lite_llama_amd.kernels.fused_moe import group_router

    torch.manual_seed(experts * 10 + top)
    n, outputs = 33, experts + identity
    h = bf(torch.randn(n, width)).to(DEV).to(dtype)
    w = bf(torch.randn(outputs, width) * 2 * width ** -0.5)
    corr = bf(torch.randn(outputs) * 0.2)      # large against the score differences: the choice differs from the plain top
    ids, weights, own = group_router(h, w.to(DEV).to(dtype), top, scoring="softmax_all", correction=corr.to(DEV).to(dtype), identity=identity)
    s = torch.softmax(d(h) @ w.to(F64).T, -1)
    want = torch.topk(s + corr.to(F64), top, dim=-1).indices
    plain = torch.topk(s, top, dim=-1).indices
    if top < outputs and outputs > 3:
        assert (want.sort(-1).values != plain.sort(-1).values).any()
    if dtype == torch.float32:
        assert (ids.cpu().long() == want).all()
    chosen = torch.gather(s, 1, ids.cpu().long())
    _close(weights, chosen, 1e-5 if dtype == torch.float32 else 1e-2)
    if identity:
        mine = (chosen * (ids.cpu() >= experts)).sum(-1)
        _close(own, mine, 1e-5 if dtype == torch.float32 else 1e-2)
        assert (ids.cpu() >= experts).any()
    else:
        assert own is None


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("experts,identity,top,width,ff,n", [(4, 2, 3, 64, 24, 19), (3, 0, 2, 36, 10, 5), (2, 1, 1, 128, 64, 600)])
def test_clamped_experts_leave_identity_slots_empty(dtype, experts, identity, top, width, ff, n):
    from lite_llama_amd.kernels.fused_moe import sparse_glu_experts
    from oracle import nivotar as O

    g = torch.Generator().manual_seed(ff)
    limit = 0.75
    h = bf(torch.randn(n, width, generator=g))
    t = {}
    for e in range(experts):
        t[f"e{e}.gate"], t[f"e{e}.up"] = bf(torch.randn(ff, width, generator=g) * 0.3), bf(torch.randn(ff, width, generator=g) * 0.3)
        t[f"e{e}.down"] = bf(torch.randn(width, ff, generator=g) * ff ** -0.5)
    ids = torch.stack([torch.randperm(experts + identity, generator=g)[:top] for _ in range(n)]).to(torch.int32)
    weights = torch.rand(n, top, generator=g)
    gu = torch.stack([torch.cat([t[f"e{e}.gate"], t[f"e{e}.up"]]) for e in range(experts)]).to(DEV).to(dtype)
    dn = torch.stack([t[f"e{e}.down"] for e in range(experts)]).to(DEV).to(dtype)
    y = sparse_glu_experts(h.to(DEV).to(dtype), gu, dn, ids.to(DEV), weights.to(DEV), limit=limit, skipped_ids=identity > 0)
    outs = [O.clamped_expert(h.to(F64), t, f"e{e}.", limit) for e in range(experts)]
    want = torch.zeros(n, top, width, dtype=F64)
    for i in range(n):
        for k in range(top):
            if ids[i, k] < experts:
                want[i, k] = weights[i, k].to(F64) * outs[int(ids[i, k])][i]
    big = torch.stack(outs).abs().max()
    assert (torch.stack([O.clamped_expert(h.to(F64), t, f"e{e}.", 1e9) for e in range(experts)]) - torch.stack(outs)).abs().max() > 0.05 * big
    _close(y, want, 2e-5 if dtype == torch.float32 else 2e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width,parts", [(96, 1), (70, 3), (2048, 2), (4100, 1), (18, 4)])
def test_result_norm_residual_add_and_plain_cast_in_one_launch(dtype, width, parts):
    """x += rmsnorm(sum of the update's rows + bias + scale * own row) * w, and the next sublayer's input is x itself, cast."""
    from lite_llama_amd.kernels.norm_act import GatedUpdate, gated_group_norm
    from oracle import nivotar as O

    torch.manual_seed(width + parts)
    n, eps = 9, 1e-6
    x = torch.randn(n, width, device=DEV)
    x0 = d(x)
    y = bf(torch.randn(n, parts, width)).to(DEV).to(dtype)
    w, b = bf(1 + 0.1 * torch.randn(width)).to(DEV).to(dtype), bf(torch.randn(width)).to(DEV).to(dtype)
    own, own_scale = bf(torch.randn(n, width)).to(DEV).to(dtype), torch.rand(n, device=DEV)
    h = gated_group_norm(x, GatedUpdate(y, w, shared=own, shared_scale=own_scale, bias=b), None, eps, plain=dtype)
    want = x0 + O.rms_norm(d(y).sum(1) + d(b) + d(own_scale)[:, None] * d(own), d(w), eps)
    _close(x, want, 3e-6)
    _close(h, want, 3e-6 if dtype == torch.float32 else 1e-2)
    first = gated_group_norm(x, None, None, eps, plain=dtype)            # (nothing pending: only the cast)
    _close(first, want, 3e-6 if dtype == torch.float32 else 1e-2)


# ------------------------------------------------------------------------------------------------------------------- #
# whole models
# ------------------------------------------------------------------------------------------------------------------- #
def _model(tmp_path_factory, name, dtype):
    from lite_llama_amd.weights import load_pretrained

    key = (name, dtype)
    if key not in _MODELS:
        cfg = T.CONFIGS[name]
        tens = T.tensors(cfg, seed=len(name))
        folder = L.write(tmp_path_factory.mktemp(name), T.on_disk(cfg), tens)
        _MODELS[key] = (load_pretrained(folder, device=DEV, dtype=dtype), T.on_disk(cfg), tens, folder)
    return _MODELS[key]


@pytest.mark.parametrize("name", sorted(T.CONFIGS))
def test_whole_prompt_layers_and_logits(tmp_path_factory, name):
    from lite_llama_amd.executor.ragged import RaggedRunner
    from oracle import nivotar as O

    model, cfg, tens, _ = _model(tmp_path_factory, name, torch.float32)
    toks = L.prompt(cfg, 45)
    want, layers = O.forward(toks, tens, cfg)
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
    decoding; pages of 8 tokens, so portions, windows, taps, token tiles and pages start and end inside one another."""
    from lite_llama_amd.executor.ragged import RaggedRunner
    from oracle import nivotar as O

    model, cfg, tens, _ = _model(tmp_path_factory, name, torch.float32)
    toks = L.prompt(cfg, 58, seed=1)
    want, _ = O.forward(toks, tens, cfg)
    runner = RaggedRunner(model, 64, 2, block_size=8, device=DEV)
    _close(_feed(runner, runner.admit(), toks, sizes), want, 2e-5)
    runner.check_errors()


@pytest.mark.parametrize("name", ["mix", "odd"])
def test_unequal_requests_in_one_batch_equal_each_alone_and_freed_pages_and_slots_are_used_again(tmp_path_factory, name):
    """Four requests of different lengths ride together in changing portions, three slots and a pool that only holds them
    because finished requests give their pages back; a late request takes over a used slot (with the state and the carried
    rows its last owner left) and used pages."""
    from lite_llama_amd.executor.ragged import RaggedRunner
    from oracle import nivotar as O

    model, cfg, tens, _ = _model(tmp_path_factory, name, torch.float32)
    lens = {"a": 41, "b": 9, "c": 26, "d": 33}
    toks = {k: L.prompt(cfg, n, seed=ord(k)) for k, n in lens.items()}
    want = {k: O.forward(v, tens, cfg)[0] for k, v in toks.items()}
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
    from oracle import nivotar as O

    model, cfg, tens, _ = _model(tmp_path_factory, name, torch.float32)
    toks = L.prompt(cfg, 150, seed=5)
    want, _ = O.forward(toks, tens, cfg)
    runner = RaggedRunner(model, 160, 1, block_size=16, device=DEV)
    _close(_feed(runner, runner.admit(), toks, [6, 1]), want, 3e-5)


@pytest.mark.parametrize("name", sorted(T.CONFIGS))
def test_bfloat16_model_tracks_the_oracle_and_its_own_portions(tmp_path_factory, name):
    from lite_llama_amd.executor.ragged import RaggedRunner
    from oracle import nivotar as O

    model, cfg, tens, _ = _model(tmp_path_factory, name, torch.bfloat16)
    toks = L.prompt(cfg, 70, seed=2)
    want, _ = O.forward(toks, tens, cfg)
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
    from oracle import nivotar as O

    model, cfg, tens, _ = _model(tmp_path_factory, "odd", torch.float32)
    prompts = [L.prompt(cfg, n, seed=n) for n in (3, 19, 1, 11, 7)]
    engine = GenerationEngine(model, max_tokens=96, max_requests=3, block_size=8, max_step_tokens=10, device=DEV)
    outs = engine.generate(prompts, SamplingParams(max_new_tokens=6))
    for p, o in zip(prompts, outs):
        assert o == O.greedy(p, 6, tens, cfg)
    captured = GenerationEngine(model, max_tokens=96, max_requests=3, block_size=8, max_step_tokens=10, device=DEV, capture_decode=True)
    assert captured.generate(prompts, SamplingParams(max_new_tokens=6)) == outs and captured.runner.replays > 0
    assert engine.runner.cache.free_blocks == engine.runner.total_blocks and engine.runner.free_slots == 3
    sampled = engine.generate(prompts[:2], SamplingParams(max_new_tokens=5, temperature=0.8, top_p=0.9, repetition_penalty=1.2))
    assert [len(s) for s in sampled] == [5, 5] and all(0 <= t < cfg["vocab"] for s in sampled for t in s)


def test_command_line_generate_and_trace_replay(tmp_path_factory, tmp_path):
    from oracle import nivotar as O

    _, cfg, tens, folder = _model(tmp_path_factory, "wide", torch.float32)
    prompt = L.prompt(cfg, 9, seed=4)
    env = dict(os.environ, PYTHONPATH=ROOT)
    done = subprocess.run([sys.executable, "-m", "lite_llama_amd", "generate", "--model", folder, "--dtype", "float32",
                           "--prompt-ids", ",".join(map(str, prompt)), "--max-new-tokens", "4"],
                          capture_output=True, text=True, env=env, cwd=ROOT, timeout=300)
    assert done.returncode == 0, done.stderr[-2000:]
    line = json.loads(done.stdout.strip().splitlines()[-1])
    assert line["prompt"] == prompt and line["generated"] == O.greedy(prompt, 4, tens, cfg)

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

    la, lb = O.forward(a, tens, cfg)[0], O.forward(b, tens, cfg)[0]
    read = lambda i: torch.from_numpy(np.fromfile(out / f"{i}.f32", dtype="<f4")).view(-1, cfg["vocab"])   # noqa: E731
    _close(read(0), la[[0, 12]], 2e-5)
    _close(read(1), lb[[5]], 2e-5)
    assert not (out / "2.f32").exists()
    _close(read(3), torch.stack([la[30], lb[5]]), 2e-5)


def _random_config(seed):
    """A configuration drawn from the whole range the reader takes: one to five layers of the three mixers in any order, head
    counts and widths with and without the matrix-core forms' multiples, windows from one key to longer than the prompt,
    rotations of a part or all of a head, one to six taps, grouped and ungrouped state-space heads, every feed-forward kind,
    with and without identity experts."""
    import random

    r = random.Random(seed)
    layers = []
    for _ in range(r.randint(1, 5)):
        kind = r.choice(["dense", "moe", None])
        experts, identity = r.randint(1, 9), r.choice([0, 0, 1, 2, 3])
        mlp = T.dense(r.choice([16, 40, 44])) if kind == "dense" else \
            T.moe(experts, identity, r.randint(1, experts + identity), r.choice([8, 12, 24]), limit=r.choice([0.5, 1.5, 30.0])) \
            if kind == "moe" else None
        mixer = r.choice(["parallel", "lightning", "gla"])
        if mixer == "parallel":
            g = r.choice([1, 2, 3])
            dim = r.choice([8, 16, 32, 64, 12, 20, 128])
            groups = r.choice([1, 2, 3])
            sh, sv = groups * r.choice([1, 2, 4]), r.choice([4, 8, 16, 10, 48])
            parts = r.choice([p for p in (1, 2, 3, 4, 6) if (sh * sv) % p == 0])
            layers.append(T.parallel(g * r.choice([1, 2, 4, 5]), g, dim, r.choice([8, 16, 24, 10, 48]),
                                     r.choice([1, 3, 8, 17, 40, 64, 200]), r.choice([dim, dim // 2, 2, max(2, (dim // 4) * 2)]),
                                     sh, sv, r.choice([4, 16, 48, 10, 128]), groups, r.randint(1, 6), parts, mlp=mlp,
                                     scale=r.choice([0.5, 1.0, 2.0]) * dim ** -0.5 * 4, base=r.choice([100.0, 10000.0, 500000.0]),
                                     left=r.choice([1.0, 0.3, 2.0]), right=r.choice([1.0, 0.5, 1.7])))
        elif mixer == "lightning":
            heads = r.randint(1, 5)
            layers.append(T.lightning(heads, r.choice([8, 16, 32, 12, 64]), r.choice([8, 16, 10, 40]),
                                      [r.choice([0.3, 0.9, 0.99, 0.998, 1.0]) for _ in range(heads)], mlp=mlp))
        else:
            layers.append(T.gla(r.randint(1, 5), r.choice([8, 16, 48, 12, 64]), r.choice([8, 16, 10, 32]), r.choice([1.0, 4.0, 32.0]),
                                r.choice([1, 4, 16, 5]), mlp=mlp))
    return T.config(layers, width=r.choice([32, 48, 60, 88]), vocab=r.randint(20, 300), eps=r.choice([1e-5, 1e-6, 1e-3]))


@pytest.mark.parametrize("seed", range(12))
def test_random_configurations_whole_in_portions_decoded_and_side_by_side(tmp_path, seed):
    from lite_llama_amd.executor.ragged import RaggedRunner
    from lite_llama_amd.weights import load_pretrained
    from oracle import nivotar as O

    cfg = _random_config(seed)
    tens = T.tensors(cfg, seed=seed)
    cfg = T.on_disk(cfg)
    model = load_pretrained(L.write(tmp_path / "m", cfg, tens), device=DEV, dtype=torch.float32)
    a, b = L.prompt(cfg, 90, seed=seed), L.prompt(cfg, 37, seed=seed + 50)
    wa, wb = O.forward(a, tens, cfg)[0], O.forward(b, tens, cfg)[0]
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
