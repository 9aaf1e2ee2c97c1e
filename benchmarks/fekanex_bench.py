"""Throughput and per-kernel roofline fractions of the Fekanex design (attention behind short convolutions with a rotation,
unit q / k norms, a window that keeps a sequence's first keys and a unit sink; clamped-GLU and softmax-over-chosen expert
feed-forwards beside the mixer under one norm; a hashed token-pair table at the input) beside the closest llama-shaped model
of the framework at equal sizes -- ``python bench.py --fekanex``.

Model level: prefill tokens/s (whole prompts in one ragged step vs. the padded-grid prefill) and decode tokens/s (one token per
sequence and step; eager and captured) for a few layers at the widths of a small production model, random weights.  Kernel
level: every kernel of the design timed alone (HIP events around a loop of launches) with its algorithmic bytes and flops, next
to the like kernel of the framework's other models at the same shape; ``far`` = how many times further from its roofline (HBM
8 TB/s or 2.5 PFLOP/s dense 16-bit MFMA, whichever bounds it) the new kernel is than its counterpart."""

from __future__ import annotations

import time

import torch

from .layered_bench import _entry, _time
from .rukedra_bench import _step_of


def kernel_table(dev, dtype, width, heads, kv_heads, dim, vdim, taps, rot, window, keep, ff, experts, top, eff, buckets,
                 prefill=(8, 512), decode=(32, 1024)):
    from lite_llama_amd.kernels import flash_attention2_no_pad, flash_decoding, skip_rmsnorm, swiglu_forward
    from lite_llama_amd.kernels.attention import conv_rope_cache, ragged_attention, rotation_table
    from lite_llama_amd.kernels.fused_moe import fused_moe, group_router, moe_route_topk, sparse_glu_experts
    from lite_llama_amd.kernels.norm_act import SummedUpdate, add_rmsnorm_shift, embed_pair, glu_act, rope_and_cache

    es = torch.empty(0, dtype=dtype).element_size()
    h16 = torch.float16 if dtype == torch.float32 else dtype
    out = []
    channels = (heads + kv_heads) * dim + kv_heads * vdim
    for phase, (batch, length) in (("prefill", prefill), ("decode", decode)):
        first, count = (0, length) if phase == "prefill" else (length - 1, 1)
        n = batch * count
        step = _step_of(dev, batch, first, count)
        ctx_rows = batch * (first + count)
        table = torch.arange(ctx_rows, dtype=torch.int32, device=dev).view(batch, first + count)
        w = torch.ones(width, device=dev, dtype=dtype)
        # input rows: embedding + pair table (+ carried previous token) vs the plain embedding lookup
        emb = torch.randn(32768, width, device=dev).to(dtype)
        pair = torch.randn(buckets + 1, width, device=dev).to(dtype)
        toks = torch.randint(0, 32768, (n,), device=dev, dtype=torch.int32)
        prev = torch.zeros(2, batch, dtype=torch.int32, device=dev)
        t_new = _time(lambda: embed_pair(toks, emb, 0.75, pair, 131, 29, step, prev))
        t_old = _time(lambda: torch.nn.functional.embedding(toks, emb))
        like = _entry("embedding lookup (one row per token, 16-bit out)", t_old, n * width * es * 2, 0)
        out.append(dict(_entry("embed_pair (two rows per token, fp32 out)", t_new, n * width * (2 * es + 4), 0, like), phase=phase))
        # residual add of a row and the experts' rows + norm vs skip_rmsnorm
        x = torch.randn(n, width, device=dev)
        for parts in (0, top):
            upd = SummedUpdate(torch.randn(n, width, device=dev).to(dtype),
                               torch.randn(n, parts, width, device=dev).to(dtype) if parts else None)
            t_new = _time(lambda: add_rmsnorm_shift(x, upd, w, 1e-6, x_out=x))
            hx, hr = upd.row.clone().to(h16), upd.row.clone().to(h16)
            t_old = _time(lambda: skip_rmsnorm(hx, hr, w.to(h16), 1e-6))
            like = _entry("skip_rmsnorm (16-bit residual)", t_old, n * width * es * 4, 0)
            out.append(dict(_entry(f"add_rmsnorm_shift (row + {parts} part rows, fp32 residual in + out)", t_new,
                                   n * width * (4 + 4 + (2 + parts) * es), 0, like), phase=phase))
        # clamped activation into a column range of the output projection's input vs swiglu
        gu = torch.randn(n, channels + 2 * ff, device=dev).to(dtype)
        mixed = torch.empty(n, heads * vdim + ff, device=dev, dtype=dtype)
        t_new = _time(lambda: glu_act(gu[:, channels:], ff, "clamped", limit=7.0, slope=1.702, out=mixed[:, heads * vdim:]))
        a, b = torch.randn(n, ff, device=dev).to(h16), torch.randn(n, ff, device=dev).to(h16)
        t_old = _time(lambda: swiglu_forward(a, b))
        like = _entry("swiglu_forward", t_old, n * ff * es * 3, 0)
        out.append(dict(_entry("glu_act (clamped, column ranges of both fused projections)", t_new, n * ff * es * 3, 0, like), phase=phase))
        # bias + convolution + rotation + unit norms + value blend + cache write vs rotation + cache write
        kc = torch.randn(ctx_rows, kv_heads, dim, device=dev).to(dtype)
        vc = torch.randn(ctx_rows, kv_heads, vdim, device=dev).to(dtype)
        src = torch.randn(ctx_rows, kv_heads, vdim, device=dev).to(dtype)
        bias = torch.randn(channels, device=dev).to(dtype)
        cw = torch.randn(channels, taps, device=dev).to(dtype)
        state = torch.zeros(2, batch, taps - 1, channels, device=dev, dtype=dtype)
        freq = torch.rand(rot // 2, device=dev)
        lam = torch.tensor([0.4], device=dev).to(dtype)
        t_tab = _time(lambda: rotation_table(step, freq, rot // 2, 1.1))
        out.append(dict(_entry("rotation_table (cos / sin per token and pair: once per step for all layers)", t_tab,
                               n * rot * 4, 0), phase=phase))
        tab = rotation_table(step, freq, rot // 2, 1.1)
        t_new = _time(lambda: conv_rope_cache(gu, heads, kv_heads, dim, vdim, step, kc, vc, bias=bias, conv_weight=cw, conv_state=state,
                                              freq=freq, pairs=rot // 2, amp=1.1, unit_norm=True, eps=1e-6, v_source=src, v_blend=lam,
                                              rot_table=tab))
        hd = 128
        qh = torch.randn(n, heads, hd, device=dev).to(h16)
        kvh = torch.randn(n, 2 * kv_heads, hd, device=dev).to(h16)
        pool = torch.zeros(ctx_rows, 2 * kv_heads, hd, device=dev, dtype=h16)
        cos = torch.randn(first + count + 8, hd // 2, device=dev).to(h16)
        pos = step.tok_pos.long()
        t_old = _time(lambda: rope_and_cache(qh, kvh, cos, cos, 1, n, step.select, pool, positions=pos))
        like = _entry("rope_and_cache (rotation + cache write)", t_old, n * (heads + 2 * kv_heads) * hd * es * 2, 0)
        moved = n * (channels * 2 + kv_heads * vdim) * es + (0 if phase == "prefill" else n * (taps - 1) * channels * es * 2)
        out.append(dict(_entry("conv_rope_cache (bias + taps + rotation + unit norms + blend + cache write + carried rows)", t_new, moved, 0,
                               like), phase=phase))
        # attention: window + kept first keys + unit sink vs the causal llama kernels at the same heads
        q = torch.randn(n, heads, dim, device=dev).to(dtype)
        sink = torch.zeros(heads, device=dev, dtype=dtype)
        wide = torch.empty(n, heads * vdim + ff, device=dev, dtype=dtype)
        qh = torch.randn(n, heads, hd, device=dev).to(h16)
        kk = torch.randn(ctx_rows, kv_heads, hd, device=dev).to(h16)
        vv = torch.randn(ctx_rows, kv_heads, hd, device=dev).to(h16)
        lens = torch.full((batch,), length, dtype=torch.int32, device=dev)
        if phase == "prefill":
            start = torch.arange(batch, dtype=torch.int32, device=dev) * length
            t_old = _time(lambda: flash_attention2_no_pad(qh, kk, vv, hd ** -0.5 * 1.4426950408889634, start, lens, length), iters=5)
            like = _entry("flash_attention2_no_pad (causal, head width 128)", t_old, n * (2 * heads + 2 * kv_heads) * hd * es,
                          batch * heads * 4.0 * hd * length * length / 2)
        else:
            req = torch.arange(batch, dtype=torch.int32, device=dev)
            t_old = _time(lambda: flash_decoding(qh, kk, vv, hd ** -0.5, table, req, lens, length))
            like = _entry("flash_decoding (causal, head width 128)", t_old, ctx_rows * 2 * kv_heads * hd * es, batch * heads * 4.0 * hd * length)
        for win, kp in ((0, 0), (window, keep)):
            name = f"ragged_attention (unit sink, {'window ' + str(win) + ' + ' + str(kp) + ' kept' if win else 'causal'})"
            t_new = _time(lambda: ragged_attention(q, kc, vc, 0.1, step, table, sink=sink, window=win, keep_first=kp,
                                                   out=wide[:, :heads * vdim]), iters=5 if phase == "prefill" else 20)
            span = min(win + kp, length) if win else length
            if phase == "prefill":
                pairs = batch * (length * span - span * (span - 1) / 2 if win else length * (length + 1) / 2)
                flops, nbytes = heads * 2.0 * (dim + vdim) * pairs, n * (heads * (dim + vdim) + kv_heads * (dim + vdim)) * es
            else:
                flops, nbytes = batch * heads * 2.0 * (dim + vdim) * span, batch * span * kv_heads * (dim + vdim) * es
            out.append(dict(_entry(name, t_new, nbytes, flops, like), phase=phase))
        # experts: router (largest logits, softmax over them) and the grouped products vs the fp16 softmax-router path
        h = torch.randn(n, width, device=dev).to(dtype)
        wr = (torch.randn(experts, width, device=dev) * width ** -0.5).to(dtype)
        t_new = _time(lambda: group_router(h, wr, top, scoring="softmax_chosen"))
        logits = torch.randn(n, experts, device=dev).to(h16)
        t_old = _time(lambda: moe_route_topk(logits, top))
        like = _entry("moe_route_topk (softmax tail only; its logits come from a library GEMM)", t_old, n * experts * es, 0)
        out.append(dict(_entry("group_router (fp32 logits + largest + softmax over the chosen)", t_new,
                               n * width * es + experts * width * es, n * experts * width * 2.0, like), phase=phase))
        ids, wts, _ = group_router(h, wr, top, scoring="softmax_chosen")
        wgu = (torch.randn(experts, 2 * eff, width, device=dev) * width ** -0.5).to(dtype)
        wd = (torch.randn(experts, width, eff, device=dev) * eff ** -0.5).to(dtype)
        t_new = _time(lambda: sparse_glu_experts(h, wgu, wd, ids, wts), iters=5)
        touched = min(experts, n * top)
        flops = n * top * 6.0 * eff * width
        nbytes = touched * 3 * eff * width * es + n * top * (width + 2 * eff + width) * es
        hf, w1, w2 = h.to(torch.float16), wgu.to(torch.float16), wd.to(torch.float16)
        t_old = _time(lambda: fused_moe(hf, w1, w2, wts.to(torch.float16), ids), iters=5)
        like = _entry("fused_moe (fp16: align + two grouped GEMMs + silu + sum)", t_old, nbytes, flops)
        out.append(dict(_entry("sparse_glu_experts (sort + gate|up with silu epilogue + weighted down)", t_new, nbytes, flops, like), phase=phase))
    return out


def _geometry(width, heads, kv_heads, dim, vdim, taps, rot, window, keep, ff, experts, top, eff, buckets, vocab, layers):
    from lite_llama_amd.model_layers import LayeredGeometry, LayerSpec, MixerSpec, MlpSpec, RotarySpec

    rotary = RotarySpec(rot, 10000.0, 8.0, 4096.0, 32.0, 1.0)
    mix = MixerSpec("conv_attention", heads=heads, dim=dim, vdim=vdim, kv_heads=kv_heads, scale=dim ** -0.5, rotary=rotary, window=window,
                    keep_first=keep, bias=True, conv_taps=taps, unit_norm=True, unit_sink=True, value_mix=True)
    dense = MlpSpec("dense", ff=ff, act="clamped", limit=7.0)
    moe = MlpSpec("moe", ff=eff, act="silu", experts=experts, top=top, scoring="softmax_chosen")
    specs = tuple(LayerSpec(mix, ff=f.ff, mlp_kind=f.kind, mlp=f) for f in ((dense, moe)[i % 2] for i in range(layers)))
    return LayeredGeometry("fekanex", vocab, width, 1e-6, specs, token_shift=False, parallel=True, embed_scale=0.75, pair_buckets=buckets,
                           pair_mul_prev=131, pair_mul_cur=29, logit_scale=1.5, tied_head=True)


def model_points(dev, dtype, geo, llama, prefill=(8, 512), decode=(32, 1024), steps=16):
    from lite_llama_amd.executor import DecodeEngine
    from lite_llama_amd.executor.ragged import RaggedRunner
    from lite_llama_amd.model import CausalLM, ModelGeometry
    from lite_llama_amd.model_layers import LayeredLM

    vocab = geo.vocab_size
    model = LayeredLM(geo, dtype=dtype).init_synthetic(0, dev)
    res = {}
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
    res["fekanex_prefill"] = {"batch": b, "prompt": length, "ms": round(dt * 1e3, 2), "tokens_per_s": round(b * length / dt)}
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
        res["fekanex_decode_captured" if captured else "fekanex_decode"] = {
            "batch": b, "ctx": ctx, "ms_per_step": round(dt * 1e3, 3), "tokens_per_s": round(b / dt),
            "launches": "one hipGraph per step" if captured else "eager"}
        runner.check_errors()
        del runner
    del model
    torch.cuda.empty_cache()
    # the closest llama-shaped model: same width, query and key/value heads (of 128), dense feed-forward width and depth; rotary
    # causal attention + swiglu in every layer
    cgeo = ModelGeometry("bench", llama["width"], len(geo.layers), llama["heads"], llama["kv_heads"], llama["hd"], llama["ff"], vocab)
    h16 = torch.float16 if dtype == torch.float32 else dtype
    cm = CausalLM(cgeo).init_synthetic(0, device=dev).to(h16)
    b, length = prefill
    eng = DecodeEngine(cm, max_batch=b, max_seq_len=length + 8, device=dev, kv_dtype=h16)
    ids = torch.randint(0, vocab, (b, length), generator=g).to(dev)
    eng.prefill(ids)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(3):
        eng.prefill(ids)
        torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / 3
    res["llama_prefill"] = {"batch": b, "prompt": length, "ms": round(dt * 1e3, 2), "tokens_per_s": round(b * length / dt)}
    del eng
    b, ctx = decode
    eng = DecodeEngine(cm, max_batch=b, max_seq_len=ctx + steps + 8, device=dev, kv_dtype=h16)
    first = eng.synthetic_context(b, ctx)
    stamps = []
    eng.decode(first, steps + 4, use_graph=True, on_step=lambda i: (torch.cuda.synchronize(), stamps.append(time.perf_counter())))
    torch.cuda.synchronize()
    dt = (time.perf_counter() - stamps[4]) / steps
    res["llama_decode"] = {"batch": b, "ctx": ctx, "ms_per_step": round(dt * 1e3, 3), "tokens_per_s": round(b / dt),
                           "launches": "one hipGraph per step"}
    return res


SIZES = {
    # widths of a 2B-class model: 16 query heads on 4 key/value heads of 128, a window of 256 keys plus 4 kept, 4 taps
    "compact": dict(width=2048, heads=16, kv_heads=4, dim=128, vdim=128, taps=4, rot=64, window=256, keep=4, ff=5632, experts=32, top=4,
                    eff=704, buckets=65521),
    # a wider model: 24 query heads on 8 key/value heads, values of 96, a window of 512 plus 16 kept, more and smaller experts
    "wide": dict(width=3072, heads=24, kv_heads=8, dim=128, vdim=96, taps=4, rot=128, window=512, keep=16, ff=8192, experts=64, top=8,
                 eff=512, buckets=262139),
}


def run(dtype_name="bf16", layers=4, sizes=("compact", "wide"), kernels=True):
    dev = torch.device("cuda", 0)
    dtype = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}[dtype_name]
    line = {"metric": "fekanex_throughput", "dtype": dtype_name, "data": "synthetic", "points": {}}
    for name in sizes:
        s = SIZES[name]
        geo = _geometry(vocab=32768, layers=layers, **s)
        llama = dict(width=s["width"], heads=s["heads"], kv_heads=s["kv_heads"], hd=128, ff=s["ff"])
        point = {"sizes": dict(s, layers=layers, vocab=32768), "model": model_points(dev, dtype, geo, llama)}
        if kernels:
            point["kernels"] = kernel_table(dev, dtype, **s)
        line["points"][name] = point
        torch.cuda.empty_cache()
    return line
