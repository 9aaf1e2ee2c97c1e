"""Small random Fekanex checkpoints for tests: configurations, tensors under the checkpoint's names (values exactly
representable in bfloat16, so a bf16 file holds the same numbers the float64 oracle reads).  Files are written with
``tests._layered.write``."""

import torch


def rot(dims, base=100.0, factor=4.0, original=64, fast=4.0, slow=0.5, scaled=True):
    out = {"base": base, "dims": dims}
    if scaled:
        out["scaling"] = {"factor": factor, "fast": fast, "original": original, "slow": slow}
    return out


def attention(heads, kv_heads, dim, vdim, conv, window, keep, rot_dims, v_mix=True, mlp=None, scale=None, **rot_kw):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": window, "keep_first": keep},
             "rot": rot(rot_dims, **rot_kw), "scale": scale if scale is not None else 3.0 * dim ** -0.5, "v_mix": v_mix}
    if conv is not None:
        mixer["conv"] = conv
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


def dense(ff, limit=1.5):
    return {"kind": "dense", "ff": ff, "limit": limit}


def moe(experts, top, ff):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def config(layers, width, vocab, buckets, mul_prev, mul_cur, scale=1.0, logit_scale=1.0, eps=1e-5):
    return {"architecture": "Fekanex", "layers": layers, "norm": {"eps": eps}, "vocab": vocab, "width": width,
            "embedding": {"scale": scale, "bigram": {"buckets": buckets, "mul_prev": mul_prev, "mul_cur": mul_cur}},
            "logit_scale": logit_scale}


CONFIGS = {
    # sizes that are multiples of 8 (the 16-bit matrix-core forms run); every feed-forward kind and a layer without one; a layer
    # that does not blend its values between layers that do; all experts chosen; windows shorter than a page, kept keys
    "mix": config([attention(4, 2, 16, 8, 4, 9, 3, 8, mlp=dense(72)),
                   attention(4, 2, 16, 8, 4, 9, 3, 8, mlp=moe(6, 2, 24)),
                   attention(2, 1, 24, 16, 2, 5, 0, 24, v_mix=False, base=37.0, factor=2.5, original=24),
                   attention(2, 2, 8, 8, 3, 12, 1, 4, mlp=moe(4, 4, 16))], width=96, vocab=83, buckets=31, mul_prev=7, mul_cur=3,
                  scale=0.25, logit_scale=3.0),
    # odd sizes: heads of 12 / 10 entries (the plain attention form), a feed-forward width that is no multiple of 8 (the
    # activation lands off a 16-byte border of the output projection's input), every head its own key/value head, the first
    # blending layer is not layer 0, one tap, no convolution at all, frequencies without scaling, one expert chosen
    "odd": config([attention(5, 5, 12, 10, 3, 4, 2, 6, v_mix=False, mlp=dense(44, limit=0.75), scaled=False),
                   attention(3, 1, 12, 10, 1, 7, 0, 12, mlp=moe(9, 1, 12), factor=8.0, original=16, fast=2.0),
                   attention(2, 1, 20, 10, None, 6, 6, 10, mlp=dense(36, limit=4.0)),
                   attention(3, 1, 12, 10, 5, 3, 1, 2)], width=60, vocab=47, buckets=13, mul_prev=40, mul_cur=11, scale=1.0,
                  logit_scale=0.5, eps=1e-6),
    # twenty heads on one key/value head (two column tiles of the grouped decode form), a window longer than a page, more kept
    # keys than a window holds, the scale 1 with a table, no scaling of the logits
    "wide": config([attention(20, 1, 8, 8, 4, 21, 5, 8, mlp=dense(40)),
                    attention(2, 2, 32, 24, 2, 6, 11, 16, v_mix=False, mlp=moe(8, 3, 8), original=512),
                    attention(20, 1, 8, 8, 6, 30, 2, 4, mlp=moe(2, 1, 16))], width=64, vocab=71, buckets=5, mul_prev=1, mul_cur=1),
    # everything that can be 1: one head of one pair, one tap, a window of one key plus one kept key, one expert of one, one
    # bucket, one layer; a width that is no multiple of 4 (rows off every 8- and 16-byte border)
    "one": config([attention(1, 1, 2, 1, 1, 1, 1, 2, mlp=moe(1, 1, 8), scale=1.0)], width=18, vocab=11, buckets=1, mul_prev=3,
                  mul_cur=5, scale=2.0, logit_scale=1.5),
}


def tensors(cfg, seed=0):
    g = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]

    def rnd(*shape, std=1.0, mean=0.0):
        return (torch.randn(*shape, generator=g) * std + mean).to(torch.bfloat16).float()

    def lin(out, inp, gain=1.0):
        return rnd(out, inp, std=gain * inp ** -0.5)

    def glu(t, p, ff):
        t[p + "gate"], t[p + "up"], t[p + "down"] = lin(ff, W, 1.5), lin(ff, W, 1.5), lin(W, ff, 1.5)

    t = {"embed": rnd(V, W), "bigram": rnd(cfg["embedding"]["bigram"]["buckets"] + 1, W, std=0.7), "final.norm": rnd(W, std=0.1, mean=1.0)}
    for i, entry in enumerate(cfg["layers"]):
        p, m = f"l{i}.", entry["mixer"]
        t[p + "norm1"] = rnd(W, std=0.1, mean=1.0)
        H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        for name, rows in (("q", H * d), ("k", G * d), ("v", G * dv)):
            t[p + "mix." + name] = lin(rows, W, 2.0)
            t[p + "mix." + name + ".b"] = rnd(rows, std=0.5)
            if m.get("conv"):
                t[p + "mix." + name + ".conv"] = rnd(rows, m["conv"], std=0.6, mean=0.3)
        if m["v_mix"]:
            t[p + "mix.vmix"] = (torch.rand((), generator=g) * 0.5 + 0.2).to(torch.bfloat16).float()
        t[p + "mix.o"] = lin(W, H * dv)
        mlp = entry["mlp"]
        if mlp is None:
            continue
        if mlp["kind"] == "dense":
            glu(t, p + "mlp.", mlp["ff"])
        else:
            t[p + "mlp.router"] = lin(mlp["router"]["experts"], W, 3.0)
            for e in range(mlp["router"]["experts"]):
                glu(t, f"{p}mlp.e{e}.", mlp["expert"]["ff"])
    return t
