"""Small random Nivotar checkpoints for tests: configurations, tensors under the checkpoint's names (values exactly
representable in bfloat16, so a bf16 file holds the same numbers the float64 oracle reads).  Files are written with
``tests._layered.write``."""

import torch


def parallel(heads, kv_heads, dim, vdim, window, rot_dims, ssd_heads, ssd_vdim, state, groups, conv, norm_groups, mlp=None,
             scale=None, base=100.0, left=0.7, right=1.2):
    return {"type": "parallel", "mlp": mlp, "mixer": {
        "left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": window},
                 "rot": {"base": base, "dims": rot_dims}, "scale": scale if scale is not None else 2.0 * dim ** -0.5},
        "right": {"heads": ssd_heads, "vdim": ssd_vdim, "state": state, "groups": groups, "conv": conv, "norm_groups": norm_groups},
        "left_scale": left, "right_scale": right}}


def lightning(heads, dim, vdim, decay, mlp=None):
    return {"type": "lightning", "mlp": mlp, "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}}


def gla(heads, dim, vdim, tau, rank, mlp=None):
    """(``rank`` is not part of a checkpoint's configuration: it is the row count of ``mix.a1`` and read from there.)"""
    return {"type": "gla", "mlp": mlp, "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau}, "_rank": rank}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, identity, top, ff, limit=2.5):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "identity": identity, "top": top}}


def config(layers, width, vocab, eps=1e-5):
    return {"architecture": "Nivotar", "layers": layers, "norm": {"eps": eps}, "vocab": vocab, "width": width}


def on_disk(cfg):
    """The configuration as a checkpoint folder holds it (without the test's bookkeeping keys)."""
    return dict(cfg, layers=[{k: v for k, v in entry.items() if not k.startswith("_")} for entry in cfg["layers"]])


CONFIGS = {
    # sizes that are multiples of 8 (the 16-bit matrix-core forms run); every mixer and feed-forward kind; a window shorter
    # than a page; grouped key/value heads and grouped state-space heads; identity experts
    "mix": config([parallel(4, 2, 16, 8, 9, 8, 4, 8, 16, 2, 4, 2, mlp=dense(72)),
                   lightning(2, 16, 24, (0.8, 0.995), mlp=moe(6, 2, 3, 24)),
                   gla(3, 16, 8, 8.0, 8, mlp=moe(4, 1, 2, 16, limit=0.75)),
                   parallel(2, 2, 24, 16, 21, 24, 2, 16, 8, 1, 2, 1)], width=96, vocab=83),
    # odd sizes: heads of 12 / 10 entries (the plain attention form), widths off every 8- and 16-byte border, every head its own
    # key/value head and its own state-space group, one tap (no carried rows), six taps, no identity experts, one expert chosen,
    # all router outputs chosen, the recurrent layers first
    "odd": config([gla(2, 12, 10, 3.0, 5, mlp=dense(44)),
                   lightning(3, 10, 6, (0.5, 0.9, 1.0)),
                   parallel(5, 5, 12, 10, 4, 6, 3, 10, 6, 3, 1, 3, mlp=moe(5, 0, 1, 12, limit=4.0)),
                   parallel(3, 1, 12, 10, 70, 12, 2, 14, 20, 1, 6, 2, mlp=moe(3, 2, 5, 20))], width=60, vocab=47, eps=1e-6),
    # twenty heads on one key/value head (two column tiles of the grouped decode form), a window longer than a page and
    # longer than the prompts, a state as wide as a matrix-core tile, a decay logit rank of one
    "wide": config([parallel(20, 1, 8, 8, 200, 4, 4, 32, 64, 2, 3, 4, mlp=moe(8, 3, 4, 8)),
                    gla(2, 64, 16, 32.0, 1, mlp=dense(40)),
                    lightning(1, 64, 64, (0.998,), mlp=moe(2, 1, 1, 16))], width=64, vocab=71),
    # everything that can be 1: one head of one pair, one state entry, a window of one key, one expert of one, one identity
    # expert, one layer of each kind; a width that is no multiple of 4
    "one": config([parallel(1, 1, 2, 1, 1, 2, 1, 1, 1, 1, 1, 1, mlp=moe(1, 1, 1, 8), scale=1.0),
                   lightning(1, 1, 1, (0.5,)), gla(1, 1, 1, 1.0, 1)], width=18, vocab=11),
}


def tensors(cfg, seed=0):
    g = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]

    def rnd(*shape, std=1.0, mean=0.0):
        return (torch.randn(*shape, generator=g) * std + mean).to(torch.bfloat16).float()

    def uni(*shape, lo=0.0, hi=1.0):
        return (torch.rand(*shape, generator=g) * (hi - lo) + lo).to(torch.bfloat16).float()

    def lin(out, inp, gain=1.0):
        return rnd(out, inp, std=gain * inp ** -0.5)

    t = {"embed": rnd(V, W), "final.norm": rnd(W, std=0.1, mean=1.0)}
    for i, entry in enumerate(cfg["layers"]):
        p, m = f"l{i}.mix.", entry["mixer"]
        t[f"l{i}.norm1"] = rnd(W, std=0.1, mean=1.0)
        if entry["type"] == "parallel":
            a, r = m["left"], m["right"]
            H, G, d, dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            t[p + "left.q"], t[p + "left.k"], t[p + "left.v"] = lin(H * d, W, 2.0), lin(G * d, W, 2.0), lin(G * dv, W)
            t[p + "left.q.norm"], t[p + "left.k.norm"] = rnd(H * d, std=0.2, mean=1.2), rnd(G * d, std=0.2, mean=1.2)
            t[p + "left.o"] = lin(W, H * dv)
            inner, gn = r["heads"] * r["vdim"], r["groups"] * r["state"]
            t[p + "right.in"] = lin(2 * inner + 2 * gn + r["heads"], W)
            t[p + "right.conv"] = rnd(inner + 2 * gn, r["conv"], std=0.6, mean=0.3)
            t[p + "right.conv.b"] = rnd(inner + 2 * gn, std=0.3)
            t[p + "right.dt_bias"] = rnd(r["heads"], std=1.0)
            t[p + "right.A_log"] = uni(r["heads"], lo=-2.0, hi=1.0)
            t[p + "right.D"] = rnd(r["heads"], std=1.0)
            t[p + "right.norm"] = rnd(inner, std=0.1, mean=1.0)
            t[p + "right.o"] = lin(W, inner)
        else:
            qk, v = m["heads"] * m["dim"], m["heads"] * m["vdim"]
            for name, rows in (("q", qk), ("k", qk), ("v", v), ("g", v)):
                t[p + name] = lin(rows, W)
            t[p + "o"] = lin(W, v)
            if entry["type"] == "lightning":
                t[p + "norm"] = rnd(v, std=0.1, mean=1.0)
            else:
                t[p + "norm"] = rnd(m["vdim"], std=0.1, mean=1.0)
                t[p + "a1"], t[p + "a2"] = lin(entry["_rank"], W), lin(qk, entry["_rank"], 2.0)
                t[p + "a2.b"] = rnd(qk, std=1.0, mean=1.0)
        mlp = entry["mlp"]
        if mlp is None:
            continue
        p = f"l{i}.mlp."
        t[f"l{i}.norm2"] = rnd(W, std=0.1, mean=1.0)
        if mlp["kind"] == "dense":
            ff = mlp["ff"]
            t[p + "gate"], t[p + "up"], t[p + "down"] = lin(ff, W, 1.5), lin(ff, W, 1.5), lin(W, ff, 1.5)
            t[p + "gate.b"], t[p + "up.b"], t[p + "down.b"] = rnd(ff, std=0.5), rnd(ff, std=0.5), rnd(W, std=0.5)
        else:
            r = mlp["router"]
            outputs = r["experts"] + r["identity"]
            t[p + "router"] = lin(outputs, W, 2.0)
            t[p + "correction"] = rnd(outputs, std=0.1)
            for e in range(r["experts"]):
                ff = mlp["expert"]["ff"]
                t[f"{p}e{e}.gate"], t[f"{p}e{e}.up"], t[f"{p}e{e}.down"] = lin(ff, W, 1.5), lin(ff, W, 1.5), lin(W, ff, 1.5)
    return t
