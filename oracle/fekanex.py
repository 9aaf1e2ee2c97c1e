"""Plain, slow restatement of the Fekanex design on the CPU, in float64 unless told otherwise: one function per mechanism,
written from the equations, consuming the checkpoint's tensor names and ``config.json`` directly.  It shares no code with
lite_llama_amd/ (no kernels, no model classes, no cache): whole sequences only, full score matrices, every expert evaluated
for every token.

Notation: T tokens, W width, H query heads, G key/value heads, d the query/key width of a head, dv its value width, taps the
length of the short convolution, E experts, eps the norm epsilon.

  * input          x_t = embed[tok_t] * scale + bigram[row_t], row_t = (tok_(t-1) * mul_prev + tok_t * mul_cur) mod buckets,
                   row_0 = buckets (the table's last row)
  * layer          h = rmsnorm(x) * w;  x <- x + (attention(h) + feed_forward(h))     (both sublayers read the same h)
  * attention      q|k|v = W h + b;  a causal convolution over time per channel;  pairs (2i, 2i + 1) of the first `dims`
                   entries of each q / k head rotated by position * f_i (YaRN-scaled f_i, cos / sin times an amplitude);  q, k
                   divided by their root mean square per head;  scores = q . k * scale over keys j <= t with
                   t - j < size or j < keep_first;  weights = exp(s) / (1 + sum exp(s));  values of layers after the first
                   value-mixing layer are (1 - lam) v + lam v_first;  W_o on the heads side by side
  * feed-forward   dense: g = min(W_g h, limit), u = clamp(W_u h, +-limit), W_d (g sigmoid(1.702 g) (u + 1))
                   experts: the `top` largest router logits, softmax over those, sum of weight * W_d(silu(W_g h) * W_u h)
  * output         logits = embed (rmsnorm(x) * w_final) * logit_scale
"""

from __future__ import annotations

import math

import torch


# ------------------------------------------------------------------------------------- #
# norms
# ------------------------------------------------------------------------------------- #
def rms_norm(x, weight, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis, times ``weight`` (``None``: no weight)."""
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if weight is None else y * weight


# ------------------------------------------------------------------------------------- #
# input
# ------------------------------------------------------------------------------------- #
def bigram_rows(tokens, bigram):
    """Row of the pair table per token: a hash of (previous token, token); the first token takes the extra last row."""
    buckets, mp, mc = int(bigram["buckets"]), int(bigram["mul_prev"]), int(bigram["mul_cur"])
    rows = [buckets]
    for prev, cur in zip(tokens[:-1], tokens[1:]):
        rows.append((int(prev) * mp + int(cur) * mc) % buckets)
    return rows


def embed(tokens, t, cfg, dtype=torch.float64):
    e = cfg["embedding"]
    x = t["embed"].to(dtype)[torch.tensor(list(tokens))] * float(e.get("scale", 1.0))
    if e.get("bigram"):
        x = x + t["bigram"].to(dtype)[torch.tensor(bigram_rows(list(tokens), e["bigram"]))]
    return x


# ------------------------------------------------------------------------------------- #
# attention
# ------------------------------------------------------------------------------------- #
def causal_conv(u, w):
    """``u [T, C]``, ``w [C, taps]``: y_t = sum_j w[:, j] u_(t - taps + 1 + j), zeros in front of the sequence."""
    T, taps = u.shape[0], w.shape[1]
    y = torch.zeros_like(u)
    for j in range(taps):
        back = taps - 1 - j
        if back < T:
            y[back:] += w[:, j] * u[:T - back]
    return y


def yarn_frequencies(rot):
    """``(f [dims / 2], amplitude)`` of ``{"base", "dims", "scaling": {factor, original, fast, slow} | None}``."""
    dims, base = int(rot["dims"]), float(rot["base"])
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    if not sc:
        return torch.tensor(f, dtype=torch.float64), 1.0
    factor, original = float(sc["factor"]), float(sc["original"])

    def dim_of(turns):
        return dims * math.log(original / (2 * math.pi * turns)) / (2 * math.log(base))

    lo = max(math.floor(dim_of(float(sc["fast"]))), 0)
    hi = min(math.ceil(dim_of(float(sc["slow"]))), dims - 1)
    out = []
    for i, fi in enumerate(f):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(fi / factor * ramp + fi * (1 - ramp))
    return torch.tensor(out, dtype=torch.float64), 0.1 * math.log(factor) + 1.0


def rotate_pairs(v, positions, rot, angle_dtype=torch.float64):
    """``v [T, heads, n]``: entry 2i with entry 2i + 1 of the first ``dims`` entries, by ``position * f_i``; the rest passes."""
    f, amp = yarn_frequencies(rot)
    dims = int(rot["dims"])
    ang = (positions.to(angle_dtype)[:, None] * f.to(angle_dtype)[None, :]).to(torch.float64)
    cos, sin = (torch.cos(ang) * amp).to(v.dtype)[:, None, :], (torch.sin(ang) * amp).to(v.dtype)[:, None, :]
    a, b = v[..., 0:dims:2], v[..., 1:dims:2]
    out = v.clone()
    out[..., 0:dims:2] = a * cos - b * sin
    out[..., 1:dims:2] = b * cos + a * sin
    return out


def visible(T, size, keep_first):
    """``[T, T]`` bool: query i sees key j when j <= i and (i - j < size or j < keep_first)."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    return (j <= i) & ((i - j < size) | (j < keep_first))


def sink_softmax(scores, mask):
    """exp(s_j) / (1 + sum over visible j of exp(s_j)): a further key with score 0 and no value sits in the denominator."""
    s = scores.masked_fill(~mask, -math.inf)
    m = torch.clamp(s.max(-1, keepdim=True).values, min=0.0)
    e = torch.exp(s - m)
    return e / (torch.exp(-m) + e.sum(-1, keepdim=True))


def attention(h, t, p, m, eps, v_first=None, angle_dtype=torch.float64):
    """One attention mixer over a whole sequence.  ``p``: the tensor prefix ``l<i>.mix.``; ``m``: the mixer's configuration.
    ``v_first``: the values of the first value-mixing layer (``None`` in that layer and without mixing).  Returns
    ``(output [T, W], values [T, G, dv])``."""
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m.get("kv_heads") or m["heads"]), int(m["dim"]), int(m["vdim"])
    out = {}
    for name in ("q", "k", "v"):
        u = h @ t[p + name].to(h.dtype).T
        if p + name + ".b" in t:
            u = u + t[p + name + ".b"].to(h.dtype)
        if m.get("conv"):
            u = causal_conv(u, t[p + name + ".conv"].to(h.dtype))
        out[name] = u
    q, k, v = out["q"].view(T, H, d), out["k"].view(T, G, d), out["v"].view(T, G, dv)
    pos = torch.arange(T)
    if m.get("rot"):
        q, k = rotate_pairs(q, pos, m["rot"], angle_dtype), rotate_pairs(k, pos, m["rot"], angle_dtype)
    q, k = rms_norm(q, None, eps), rms_norm(k, None, eps)
    if v_first is not None:
        lam = t[p + "vmix"].to(h.dtype)
        v = (1 - lam) * v + lam * v_first
    mask_cfg = m.get("mask") or {}
    mask = visible(T, int(mask_cfg.get("size") or T + 1), int(mask_cfg.get("keep_first") or 0))
    heads = []
    for a in range(H):
        g = a // (H // G)
        w = sink_softmax(q[:, a] @ k[:, g].T * float(m["scale"]), mask)
        heads.append(w @ v[:, g])
    return torch.cat(heads, -1) @ t[p + "o"].to(h.dtype).T, v


# ------------------------------------------------------------------------------------- #
# feed-forwards
# ------------------------------------------------------------------------------------- #
def clamped_glu(h, t, p, limit):
    g = torch.clamp(h @ t[p + "gate"].to(h.dtype).T, max=limit)
    u = torch.clamp(h @ t[p + "up"].to(h.dtype).T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1)) @ t[p + "down"].to(h.dtype).T


def route(h, router, top):
    """``(ids [T, top], weights [T, top])``: the largest logits and the softmax over them alone."""
    z = h @ router.to(h.dtype).T
    val, ids = torch.topk(z, top, dim=-1)
    return ids, torch.softmax(val, -1)


def moe(h, t, p, mlp):
    E, top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
    ids, w = route(h, t[p + "router"], top)
    y = torch.zeros(h.shape[0], t[p + "e0.down"].shape[0], dtype=h.dtype)
    for e in range(E):
        q = f"{p}e{e}."
        z = h @ t[q + "gate"].to(h.dtype).T
        ye = (z * torch.sigmoid(z) * (h @ t[q + "up"].to(h.dtype).T)) @ t[q + "down"].to(h.dtype).T
        y = y + ye * ((ids == e) * w).sum(-1, keepdim=True)
    return y


def feed_forward(h, t, p, mlp):
    if mlp is None:
        return torch.zeros_like(h)
    if mlp.get("kind", "dense") == "dense":
        return clamped_glu(h, t, p, float(mlp["limit"]))
    return moe(h, t, p, mlp)


# ------------------------------------------------------------------------------------- #
# the model
# ------------------------------------------------------------------------------------- #
def forward(tokens, t, cfg, dtype=torch.float64, angle_dtype=torch.float64, layers_out: list | None = None):
    """Logits ``[T, vocab]`` of one whole sequence.  ``layers_out`` receives the residual stream after every layer."""
    eps = float(cfg["norm"]["eps"])
    x = embed(tokens, t, cfg, dtype)
    v_first = None
    for i, entry in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = rms_norm(x, t[p + "norm1"].to(dtype), eps)
        m = entry["mixer"]
        mixes = bool(m.get("v_mix"))
        y, v = attention(h, t, p + "mix.", m, eps, v_first if mixes else None, angle_dtype)
        if mixes and v_first is None:
            v_first = v
        x = x + (y + feed_forward(h, t, p + "mlp.", entry.get("mlp")))
        if layers_out is not None:
            layers_out.append(x.clone())
    h = rms_norm(x, t["final.norm"].to(dtype), eps)
    return h @ t["embed"].to(dtype).T * float(cfg.get("logit_scale", 1.0))


def greedy(prompt, t, cfg, new_tokens, dtype=torch.float64):
    """Greedy continuation by recomputing the whole sequence per token."""
    seq, out = list(prompt), []
    for _ in range(new_tokens):
        nxt = int(forward(seq, t, cfg, dtype)[-1].argmax())
        seq.append(nxt)
        out.append(nxt)
    return out
