"""Throughput and per-kernel roofline fractions of the Nivotar design (windowed attention with whole-row q / k norms beside a
state-space mixer; linear attention with a fixed decay per head and with a decay per key entry; biased silu and corrected-softmax
expert feed-forwards; the norm on every sublayer's result) beside the closest model of the framework at equal sizes -- the
layered family's Rakevik (softmax attention + HGRN2 recurrences + dense feed-forwards over the same ragged runner, paged state
cache and fp32 residual stream) -- ``python bench.py --nivotar``.

Model level: prefill tokens/s (whole prompts in one ragged step) and decode tokens/s (one token per sequence and step; eager
and captured) for four layers at the widths of a small production model, random weights.  Kernel level: every new kernel of the
design timed alone (HIP events around a loop of launches) with its algorithmic bytes and flops, next to the like kernel of the
framework's other models at the same shape; ``far`` = how many times further from its roofline (HBM 8 TB/s or 2.5 PFLOP/s dense
16-bit MFMA, whichever bounds it) the new kernel is than its counterpart."""

from __future__ import annotations

import time

import torch

from .layered_bench import _entry, _time
from .rukedra_bench import _step_of


def kernel_table(dev, dtype, width, heads, kv_heads, dim, vdim, rot, window, ssd_heads, ssd_vdim, state, groups, taps, parts,
                 lin_heads, lin_dim, lin_vdim, gla_heads, gla_dim, gla_vdim, rank, ff, experts, identity, top, eff,
                 prefill=(8, 512), decode=(32, 1024)):
    from lite_llama_amd.kernels.attention import conv_rope_cache, qk_norm_cache, rownorm_rope_cache
    from lite_llama_amd.kernels.fused_moe import group_router
    from lite_llama_amd.kernels.norm_act import GatedUpdate, add_rmsnorm_shift, gated_group_norm
    from lite_llama_amd.kernels.recurrent import conv_act, gated_linear_scan, gated_out_norm, linear_scan

    es = torch.empty(0, dtype=dtype).element_size()
    out = []
    rnd = lambda *shape: torch.randn(*shape, device=dev).to(dtype)   # noqa: E731
    for phase, (batch, length) in (("prefill", prefill), ("decode", decode)):
        first, count = (0, length) if phase == "prefill" else (length - 1, 1)
        n = batch * count
        step = _step_of(dev, batch, first, count)
        ctx_rows = batch * (first + count)
        iters = 5 if phase == "prefill" else 20

        # the three decays of the scan (+ the read-out norm) vs the HGRN2 scan (+ its head norm) at the same head geometry
        def like_scan(h, dk, dv):
            rows = rnd(n, 2 * h * dk + h * dv) * 0.3
            st = torch.zeros(batch, h, dk, dv, device=dev)
            fb, lo, nw = rnd(h * dk), torch.rand(h * dk, device=dev).to(dtype), rnd(dv)
            t = _time(lambda: gated_linear_scan(rows, h, dk, dv, fb, lo, nw, 1e-6, step, st), iters=iters)
            moved = n * (2 * h * dk + 2 * h * dv) * es + (2 if phase == "decode" else 0) * batch * h * dk * dv * 4
            return _entry(f"gated_linear_scan + head norm (HGRN2, {h} x {dk} x {dv})", t, moved, n * h * 4.0 * dk * dv)

        def scan_row(name, h, dk, dv, qk_heads, extra_cols, call, norm):
            rows = rnd(n, 2 * qk_heads * dk + 2 * h * dv + extra_cols) * 0.3
            st = torch.zeros(batch, h, dk, dv, device=dev)
            t = _time(lambda: norm(call(rows, st), rows), iters=iters)
            moved = n * (2 * qk_heads * dk + 3 * h * dv + extra_cols) * es + (2 if phase == "decode" else 0) * batch * h * dk * dv * 4
            out.append(dict(_entry(name, t, moved, n * h * 4.0 * dk * dv, like_scan(h, dk, dv)), phase=phase))

        h, dk, dv = lin_heads, lin_dim, lin_vdim
        qk, vw = h * dk, h * dv
        dec = torch.rand(h, device=dev) * 0.1 + 0.9
        w_all = rnd(vw)
        scan_row(f"linear_scan (fixed decay, silu features) + gated_out_norm ({h} x {dk} x {dv})", h, dk, dv, h, 0,
                 lambda r, st: linear_scan(r[:, :qk], r[:, qk:2 * qk], r[:, 2 * qk:2 * qk + vw], h, dk, dv, step, st, act=True, head_decay=dec),
                 lambda o, r: gated_out_norm(o, w_all, 1e-6, gate=r[:, 2 * qk + vw:], gate_kind="sigmoid"))
        h2, dk2, dv2 = gla_heads, gla_dim, gla_vdim
        qk2, vw2 = h2 * dk2, h2 * dv2
        gb, w_head = rnd(qk2), rnd(dv2)
        scan_row(f"linear_scan (decay per key entry) + gated_out_norm ({h2} x {dk2} x {dv2})", h2, dk2, dv2, h2, qk2,
                 lambda r, st: linear_scan(r[:, :qk2], r[:, qk2:2 * qk2], r[:, 2 * qk2:2 * qk2 + vw2], h2, dk2, dv2, step, st,
                                           q_scale=dk2 ** -0.5, gate=r[:, 2 * qk2 + 2 * vw2:], gate_bias=gb, tau=8.0),
                 lambda o, r: gated_out_norm(o, w_head, 1e-6, parts=h2, gate=r[:, 2 * qk2 + vw2:2 * qk2 + 2 * vw2], gate_kind="silu"))
        h3, dk3, dv3 = ssd_heads, state, ssd_vdim
        gn, vw3 = groups * state, ssd_heads * ssd_vdim
        vecs = [rnd(h3) * 0.5 for _ in range(3)]
        w_in = rnd(vw3)
        scan_row(f"linear_scan (decay per head and token, {groups} groups) + gated_out_norm ({h3} x {dk3} x {dv3})", h3, dk3, dv3, groups, h3,
                 lambda r, st: linear_scan(r[:, :gn], r[:, gn:2 * gn], r[:, 2 * gn:2 * gn + vw3], h3, dk3, dv3, step, st, qk_heads=groups,
                                           dt=r[:, 2 * gn + 2 * vw3:], dt_bias=vecs[0], a_log=vecs[1], skip=vecs[2]),
                 lambda o, r: gated_out_norm(o, w_in, 1e-6, parts=parts, gate=r[:, 2 * gn + vw3:2 * gn + 2 * vw3], gate_kind="silu",
                                             gate_first=True, scale=1.5))
        o32 = torch.randn(n, vw, device=dev)
        gate = rnd(n, vw)
        t = _time(lambda: gated_out_norm(o32, w_all, 1e-6, gate=gate, gate_kind="sigmoid"))
        out.append(dict(_entry("gated_out_norm alone (fp32 read-out in, one part)", t, n * vw * (4 + 2 * es), 0), phase=phase))

        # causal convolution + silu with carried rows vs the attention-side convolution kernel (which also rotates and caches)
        channels = vw3 + 2 * gn
        rows = rnd(n, channels + 64)
        cw, cb = rnd(channels, taps), rnd(channels)
        cstate = torch.zeros(2, batch, taps - 1, channels, device=dev, dtype=dtype)
        t_new = _time(lambda: conv_act(rows[:, 64:], cw, cb, step, cstate))
        ch, ckv, cd = max(channels // 128 - 2, 1), 1, 128
        like_rows = rnd(n, (ch + 2 * ckv) * cd)
        lkc, lvc = rnd(ctx_rows, ckv, cd), rnd(ctx_rows, ckv, cd)
        lw, lb = rnd((ch + 2 * ckv) * cd, taps), rnd((ch + 2 * ckv) * cd)
        lstate = torch.zeros(2, batch, taps - 1, (ch + 2 * ckv) * cd, device=dev, dtype=dtype)
        t_old = _time(lambda: conv_rope_cache(like_rows, ch, ckv, cd, cd, step, lkc, lvc, bias=lb, conv_weight=lw, conv_state=lstate))
        like = _entry(f"conv_rope_cache (bias + taps + cache write, {(ch + 2 * ckv) * cd} channels)", t_old, n * (ch + 2 * ckv) * cd * es * 2, 0)
        out.append(dict(_entry(f"conv_act (bias + {taps} taps + silu + carried rows, {channels} channels)", t_new, n * channels * es * 2, 0, like),
                        phase=phase))

        # whole-row norms + half-split rotation + cache write vs per-head norms + cache write
        qkv = rnd(n, (heads + kv_heads) * dim + kv_heads * vdim)
        kc, vc = rnd(ctx_rows, kv_heads, dim), rnd(ctx_rows, kv_heads, vdim)
        qw, kw = rnd(heads * dim), rnd(kv_heads * dim)
        freq = torch.rand(rot // 2, device=dev)
        t_new = _time(lambda: rownorm_rope_cache(qkv, heads, kv_heads, dim, vdim, step, kc, vc, q_weight=qw, k_weight=kw, eps=1e-6, freq=freq,
                                                 pairs=rot // 2, value_scale=0.5))
        hw = rnd(dim)
        t_old = _time(lambda: qk_norm_cache(qkv, heads, kv_heads, dim, vdim, hw, hw, 1e-6, 0.1, 64, step, kc, vc))
        moved = n * ((heads + kv_heads) * dim + kv_heads * vdim) * es * 2
        like = _entry("qk_norm_cache (per-head norms + position temperature + cache write)", t_old, moved, 0)
        out.append(dict(_entry("rownorm_rope_cache (whole-row norms + rotation + cache write)", t_new, moved, 0, like), phase=phase))

        # result norm + residual add + plain cast vs residual add + norm
        x = torch.randn(n, width, device=dev)
        w = rnd(width)
        for slots in (1, top):
            upd = GatedUpdate(rnd(n, slots, width), w, shared=rnd(n, width) if slots > 1 else None,
                              shared_scale=torch.rand(n, device=dev) if slots > 1 else None, bias=w if slots == 1 else None)
            t_new = _time(lambda: gated_group_norm(x, upd, None, 1e-6, plain=dtype))
            row = rnd(n, width)
            t_old = _time(lambda: add_rmsnorm_shift(x, row, w, 1e-6, x_out=x))
            like = _entry("add_rmsnorm_shift (row, fp32 residual in + out)", t_old, n * width * (8 + 2 * es), 0)
            out.append(dict(_entry(f"gated_group_norm (norm of {slots} result rows{' + own row' if slots > 1 else ' + bias'}, add, plain cast)",
                                   t_new, n * width * (8 + (slots + 1 + (slots > 1)) * es), 0, like), phase=phase))

        # router: softmax over all outputs, corrected choice, identity outputs vs the largest-logits router
        hh = rnd(n, width)
        wr = rnd(experts + identity, width) * width ** -0.5
        corr = rnd(experts + identity) * 0.01
        t_new = _time(lambda: group_router(hh, wr, top, scoring="softmax_all", correction=corr, identity=identity))
        t_old = _time(lambda: group_router(hh, wr, top, scoring="softmax_chosen"))
        moved, flops = (n + experts + identity) * width * es, n * (experts + identity) * width * 2.0
        like = _entry("group_router (largest logits, softmax over the chosen)", t_old, moved, flops)
        out.append(dict(_entry("group_router (softmax over all, corrected choice, identity outputs)", t_new, moved, flops, like), phase=phase))
    return out


def _geometries(width, heads, kv_heads, dim, vdim, rot, window, ssd_heads, ssd_vdim, state, groups, taps, parts, lin_heads, lin_dim,
                lin_vdim, gla_heads, gla_dim, gla_vdim, rank, ff, experts, identity, top, eff, vocab):
    """``(the Nivotar stack, the closest Rakevik stack)``: parallel + dense, lightning + experts, gla + experts, gla + experts
    beside attention + dense, and three HGRN2 layers with dense feed-forwards of the same head geometry."""
    from lite_llama_amd.model_layers import LayeredGeometry, LayerSpec, MixerSpec, MlpSpec, RotarySpec, StateSpaceSpec

    ssd = StateSpaceSpec(ssd_heads, ssd_vdim, state, groups, taps, parts)
    par = MixerSpec("attention_ssd", heads=heads, dim=dim, vdim=vdim, kv_heads=kv_heads, scale=dim ** -0.5, rotary=RotarySpec(rot, 10000.0),
                    window=window, ssd=ssd, branch_scales=(0.5, 1.5))
    lin = MixerSpec("decay_linear", heads=lin_heads, dim=lin_dim, vdim=lin_vdim,
                    decay=tuple(1.0 - 2.0 ** -(5 + 3 * i / max(lin_heads - 1, 1)) for i in range(lin_heads)))
    gla = MixerSpec("gla", heads=gla_heads, dim=gla_dim, vdim=gla_vdim, tau=8.0, decay_rank=rank)
    dense = MlpSpec("dense", ff=ff, act="silu", bias=True)
    moe = MlpSpec("moe", ff=eff, act="clamped", limit=7.0, experts=experts, top=top, scoring="softmax_all", identity=identity)
    new = LayeredGeometry("nivotar", vocab, width, 1e-6, tuple(LayerSpec(m, ff=f.ff, mlp_kind=f.kind, mlp=f) for m, f in
                                                              ((par, dense), (lin, moe), (gla, moe), (gla, moe))),
                          token_shift=False, tied_head=True, post_norm=True)
    att = MixerSpec("attention", heads=heads, dim=dim, vdim=vdim, kv_heads=kv_heads, scale=dim ** -0.5, temp_coef=0.1, temp_every=64)
    old = LayeredGeometry("rakevik", vocab, width, 1e-6,
                          (LayerSpec(att, ff=ff), LayerSpec(MixerSpec("hgrn2", lin_heads, lin_dim, lin_vdim), ff=ff),
                           LayerSpec(MixerSpec("hgrn2", gla_heads, gla_dim, gla_vdim), ff=ff),
                           LayerSpec(MixerSpec("hgrn2", gla_heads, gla_dim, gla_vdim), ff=ff)))
    return new, old


def model_points(dev, dtype, geos, prefill=(8, 512), decode=(32, 1024), steps=16):
    from lite_llama_amd.executor.ragged import RaggedRunner
    from lite_llama_amd.model_layers import LayeredLM

    res = {}
    for label, geo in zip(("nivotar", "rakevik"), geos):
        vocab = geo.vocab_size
        model = LayeredLM(geo, dtype=dtype).init_synthetic(0, dev)
        g = torch.Generator().manual_seed(5)
        b, length = prefill
        runner = RaggedRunner(model, b * (length + 64), b, 64, dev)
        prompts = [torch.randint(0, vocab, (length,), generator=g).tolist() for _ in range(b)]

        def run_prefill():
            slots = [runner.admit() for _ in range(b)]
            runner.step(list(zip(slots, prompts)))
            torch.cuda.synchronize()
            runner.release(slots)

        run_prefill()
        t0 = time.perf_counter()
        for _ in range(3):
            run_prefill()
        dt = (time.perf_counter() - t0) / 3
        res[f"{label}_prefill"] = {"batch": b, "prompt": length, "ms": round(dt * 1e3, 2), "tokens_per_s": round(b * length / dt)}
        del runner
        b, ctx = decode
        for captured in (False, True):
            runner = RaggedRunner(model, b * (ctx + 64), b, 64, dev, capture_decode=captured)
            slots = [runner.admit() for _ in range(b)]
            for lo in range(0, ctx, 256):
                runner.step([(s, torch.randint(0, vocab, (min(256, ctx - lo),), generator=g).tolist()) for s in slots], [])
            toks = [[1]] * b
            for _ in range(3):
                runner.step(list(zip(slots, toks)))
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(steps):
                runner.step(list(zip(slots, toks)))
            torch.cuda.synchronize()
            dt = (time.perf_counter() - t0) / steps
            res[f"{label}_decode_captured" if captured else f"{label}_decode"] = {
                "batch": b, "ctx": ctx, "ms_per_step": round(dt * 1e3, 3), "tokens_per_s": round(b / dt),
                "launches": "one hipGraph per step" if captured else "eager"}
            runner.check_errors()
            del runner
        del model
        torch.cuda.empty_cache()
    return res


SIZES = {
    # widths of a 2B-class model: 16 query heads on 4 key/value heads of 128 with a window of 512 beside 32 state-space heads of 64
    # over a state of 128; 16 linear-attention heads of 128 x 128; 8 gated heads of 128 x 256; 32 + 2 experts, 4 chosen
    "compact": dict(width=2048, heads=16, kv_heads=4, dim=128, vdim=128, rot=64, window=512, ssd_heads=32, ssd_vdim=64, state=128, groups=4,
                    taps=4, parts=4, lin_heads=16, lin_dim=128, lin_vdim=128, gla_heads=8, gla_dim=128, gla_vdim=256, rank=16, ff=5632,
                    experts=32, identity=2, top=4, eff=704),
    # a wider model: 24 query heads on 8 key/value heads with values of 96, 48 state-space heads, more and smaller experts
    "wide": dict(width=3072, heads=24, kv_heads=8, dim=128, vdim=96, rot=128, window=1024, ssd_heads=48, ssd_vdim=64, state=64, groups=8,
                 taps=4, parts=8, lin_heads=24, lin_dim=64, lin_vdim=128, gla_heads=12, gla_dim=128, gla_vdim=256, rank=32, ff=8192,
                 experts=64, identity=4, top=8, eff=512),
}


def run(dtype_name="bf16", sizes=("compact", "wide"), kernels=True):
    dev = torch.device("cuda", 0)
    dtype = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}[dtype_name]
    line = {"metric": "nivotar_throughput", "dtype": dtype_name, "data": "synthetic", "points": {}}
    for name in sizes:
        s = SIZES[name]
        point = {"sizes": dict(s, layers=4, vocab=32768), "model": model_points(dev, dtype, _geometries(vocab=32768, **s))}
        if kernels:
            point["kernels"] = kernel_table(dev, dtype, **s)
        line["points"][name] = point
        torch.cuda.empty_cache()
    return line
