"""Plain, slow restatement of the Nivotar design on the CPU, in float64 unless told otherwise: one function per mechanism,
written from the equations, consuming the checkpoint's tensor names and ``config.json`` directly.  It shares no code with
lite_llama_amd/ (no kernels, no model classes, no cache): whole sequences only, full score matrices, token loops for every
recurrence, every expert evaluated for every token.

Notation: T tokens, W width, H heads (G key/value heads or groups), d the query/key width of a head, dv its value width,
N the state width of the state-space mixer, E experts, I identity experts, eps the norm epsilon.

  * layer       x <- x + rmsnorm(mixer(x)) w_1;  x <- x + rmsnorm(ff(x)) w_2      (sublayers read x itself; the norm sits on
                the sublayer's RESULT)
  * parallel    a_l * attention(x) + a_r * ssd(x)
      attention   q, k, v = W x;  q and k RMS-normed over their WHOLE row (all heads at once) with a weight per entry;  entry i
                  of a head's first `dims` entries is rotated with entry i + dims / 2 by position * base^(-2 i / dims);  scores
                  q . k * scale over keys j with 0 <= t - j < size;  softmax;  W_o over the heads side by side
      ssd         W_in x = [z | u | B | C | dt];  u, B, C through a causal convolution per channel (+ bias) and silu;
                  dt = softplus(dt + dt_bias);  per head S <- exp(-exp(A_log) dt) S + dt B u^T,  y = S^T C + D u;
                  y silu(z), RMS-normed in equal parts, times a weight, W_o
  * lightning   q, k, v = silu(W x);  per head S <- decay_h S + k v^T,  o = S^T q;  the heads side by side RMS-normed together,
                times sigmoid(W_g x), W_o
  * gla         q = W_q x / sqrt(d), k, v = W x;  alpha = sigmoid(W_a2 W_a1 x + b)^(1 / tau) per key entry;
                S <- diag(alpha) S + k v^T,  o = S^T q;  every head RMS-normed with one weight [dv], times silu(W_g x), W_o
  * dense ff    W_d (silu(W_g x + b_g) (W_u x + b_u)) + b_d
  * experts     s = softmax(W_r x) over E + I outputs;  the `top` largest s + correction are chosen;  sum of s_e expert_e(x),
                expert(x) = W_d (g sigmoid(1.702 g) (u + 1)), g = min(W_g x, limit), u = clamp(W_u x, +-limit);  the last I
                outputs stand for experts that return x itself
  * output      logits = embed (rmsnorm(x) w_f)
"""

from __future__ import annotations

import math

import torch


def rms_norm(x, weight, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis, times ``weight`` (``None``: no weight)."""
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def silu(x):
    return x * torch.sigmoid(x)


def softplus(x):
    return torch.where(x > 30.0, x, torch.log1p(torch.exp(torch.clamp(x, max=30.0))))


# ------------------------------------------------------------------------------------- #
# softmax attention with a window
# ------------------------------------------------------------------------------------- #
def rotate_half(x, positions, dims, base):
    """``x [T, heads, d]``: entry i < dims / 2 of every head paired with entry i + dims / 2."""
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=torch.float64).to(x.dtype)
    ang = positions.to(x.dtype)[:, None] * f[None, :]
    cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    out = x.clone()
    a, b = x[..., :half], x[..., half:dims]
    out[..., :half] = a * cos - b * sin
    out[..., half:dims] = b * cos + a * sin
    return out


def visible(T, size):
    """``[T, T]`` bool: query t sees key j when 0 <= t - j < size."""
    t = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    return (j <= t) & (t - j < size)


def window_attention(x, t, p, m, eps):
    """``p``: the tensor prefix of this attention (``l<i>.mix.left.``)."""
    T = x.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    dt = x.dtype
    q = rms_norm(x @ t[p + "q"].to(dt).T, t[p + "q.norm"].to(dt), eps).view(T, H, d)
    k = rms_norm(x @ t[p + "k"].to(dt).T, t[p + "k.norm"].to(dt), eps).view(T, G, d)
    v = (x @ t[p + "v"].to(dt).T).view(T, G, dv)
    pos = torch.arange(T)
    rot = m.get("rot")
    if rot:
        q = rotate_half(q, pos, int(rot["dims"]), float(rot["base"]))
        k = rotate_half(k, pos, int(rot["dims"]), float(rot["base"]))
    mask = visible(T, int(m["mask"]["size"]))
    heads = []
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * float(m["scale"])
        s = s.masked_fill(~mask, -math.inf)
        heads.append(torch.softmax(s, dim=-1) @ v[:, g])
    return torch.cat(heads, dim=-1) @ t[p + "o"].to(dt).T


# ------------------------------------------------------------------------------------- #
# state-space mixer (scalar decay per head and token)
# ------------------------------------------------------------------------------------- #
def causal_conv(u, w, b):
    """``u [T, C]``, ``w [C, taps]``: y_t = b + sum_j w[:, j] u_(t - taps + 1 + j), zeros in front of the sequence."""
    T, taps = u.shape[0], w.shape[1]
    y = torch.zeros_like(u) + b
    for j in range(taps):
        back = taps - 1 - j
        if back < T:
            y[back:] += w[:, j] * u[:T - back]
    return y


def decay_scan(q, k, v, a):
    """One head, token by token: S <- diag(a_t) S + k_t v_t^T, o_t = S^T q_t.  ``q, k [T, d]``, ``v [T, dv]``, ``a [T, d]`` (or
    anything that broadcasts to it: ``[T, 1]``, a number).  Returns ``(o [T, dv], the last S)``."""
    T, d = k.shape
    a = torch.as_tensor(a, dtype=q.dtype) * torch.ones(T, d, dtype=q.dtype)
    S = torch.zeros(d, v.shape[1], dtype=q.dtype)
    o = torch.zeros(T, v.shape[1], dtype=q.dtype)
    for i in range(T):
        S = a[i][:, None] * S + torch.outer(k[i], v[i])
        o[i] = S.T @ q[i]
    return o, S


def ssd(x, t, p, m, eps):
    T, dt_ = x.shape[0], x.dtype
    H, dv, N, G = int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m["groups"])
    inner = H * dv
    rows = x @ t[p + "in"].to(dt_).T
    z, xbc, dt = rows[:, :inner], rows[:, inner:2 * inner + 2 * G * N], rows[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, t[p + "conv"].to(dt_), t[p + "conv.b"].to(dt_)))
    u = xbc[:, :inner].view(T, H, dv)
    B = xbc[:, inner:inner + G * N].view(T, G, N)
    C = xbc[:, inner + G * N:].view(T, G, N)
    dt = softplus(dt + t[p + "dt_bias"].to(dt_))
    rate = torch.exp(t[p + "A_log"].to(dt_))
    D = t[p + "D"].to(dt_)
    y = torch.zeros(T, H, dv, dtype=dt_)
    for h in range(H):
        g = h // (H // G)
        o, _ = decay_scan(C[:, g], B[:, g], dt[:, h, None] * u[:, h], torch.exp(-rate[h] * dt[:, h, None]))
        y[:, h] = o + D[h] * u[:, h]
    y = y.view(T, inner) * silu(z)
    parts = int(m["norm_groups"])
    y = rms_norm(y.view(T, parts, inner // parts), None, eps).view(T, inner) * t[p + "norm"].to(dt_)
    return y @ t[p + "o"].to(dt_).T


def parallel(x, t, p, m, eps):
    return float(m["left_scale"]) * window_attention(x, t, p + "left.", m["left"], eps) \
        + float(m["right_scale"]) * ssd(x, t, p + "right.", m["right"], eps)


# ------------------------------------------------------------------------------------- #
# linear attention with a fixed decay per head / with a decay per key entry
# ------------------------------------------------------------------------------------- #
def lightning(x, t, p, m, eps):
    T, dt = x.shape[0], x.dtype
    H, d, dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    q = silu(x @ t[p + "q"].to(dt).T).view(T, H, d)
    k = silu(x @ t[p + "k"].to(dt).T).view(T, H, d)
    v = silu(x @ t[p + "v"].to(dt).T).view(T, H, dv)
    o = torch.zeros(T, H, dv, dtype=dt)
    for h in range(H):
        o[:, h], _ = decay_scan(q[:, h], k[:, h], v[:, h], float(m["decay"][h]))
    o = rms_norm(o.view(T, H * dv), t[p + "norm"].to(dt), eps) * torch.sigmoid(x @ t[p + "g"].to(dt).T)
    return o @ t[p + "o"].to(dt).T


def gla(x, t, p, m, eps):
    T, dt = x.shape[0], x.dtype
    H, d, dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    q = (x @ t[p + "q"].to(dt).T).view(T, H, d) * d ** -0.5
    k = (x @ t[p + "k"].to(dt).T).view(T, H, d)
    v = (x @ t[p + "v"].to(dt).T).view(T, H, dv)
    zed = (x @ t[p + "a1"].to(dt).T) @ t[p + "a2"].to(dt).T + t[p + "a2.b"].to(dt)
    alpha = torch.exp(torch.nn.functional.logsigmoid(zed) / float(m["tau"])).view(T, H, d)
    o = torch.zeros(T, H, dv, dtype=dt)
    for h in range(H):
        o[:, h], _ = decay_scan(q[:, h], k[:, h], v[:, h], alpha[:, h])
    o = rms_norm(o, t[p + "norm"].to(dt), eps).view(T, H * dv) * silu(x @ t[p + "g"].to(dt).T)
    return o @ t[p + "o"].to(dt).T


MIXERS = {"parallel": parallel, "lightning": lightning, "gla": gla}


# ------------------------------------------------------------------------------------- #
# feed-forwards
# ------------------------------------------------------------------------------------- #
def dense_mlp(x, t, p):
    dt = x.dtype
    g = x @ t[p + "gate"].to(dt).T + t[p + "gate.b"].to(dt)
    u = x @ t[p + "up"].to(dt).T + t[p + "up.b"].to(dt)
    return (silu(g) * u) @ t[p + "down"].to(dt).T + t[p + "down.b"].to(dt)


def clamped_expert(x, t, p, limit):
    dt = x.dtype
    g = torch.clamp(x @ t[p + "gate"].to(dt).T, max=limit)
    u = torch.clamp(x @ t[p + "up"].to(dt).T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ t[p + "down"].to(dt).T


def route(x, t, p, r):
    """``(ids [T, top], weights [T, top])``: chosen by score + correction, weighted by the score alone."""
    s = torch.softmax(x @ t[p + "router"].to(x.dtype).T, dim=-1)
    choice = s + t[p + "correction"].to(x.dtype)
    ids = torch.topk(choice, int(r["top"]), dim=-1).indices
    return ids, torch.gather(s, 1, ids)


def moe(x, t, p, mlp):
    r = mlp["router"]
    E = int(r["experts"])
    ids, w = route(x, t, p, r)
    outs = [clamped_expert(x, t, f"{p}e{e}.", float(mlp["expert"]["limit"])) for e in range(E)]
    y = torch.zeros_like(x)
    for i in range(x.shape[0]):
        for e, we in zip(ids[i].tolist(), w[i]):
            y[i] += we * (outs[e][i] if e < E else x[i])
    return y


# ------------------------------------------------------------------------------------- #
# the model
# ------------------------------------------------------------------------------------- #
def forward(tokens, t, cfg, dtype=torch.float64):
    """``(logits [T, vocab], residual stream after every layer [layers, T, W])`` of one whole sequence."""
    eps = float(cfg["norm"]["eps"])
    x = t["embed"].to(dtype)[torch.tensor(list(tokens))]
    layers = []
    for i, entry in enumerate(cfg["layers"]):
        p = f"l{i}."
        x = x + rms_norm(MIXERS[entry["type"]](x, t, p + "mix.", entry["mixer"], eps), t[p + "norm1"].to(dtype), eps)
        mlp = entry.get("mlp")
        if mlp is not None:
            y = dense_mlp(x, t, p + "mlp.") if mlp["kind"] == "dense" else moe(x, t, p + "mlp.", mlp)
            x = x + rms_norm(y, t[p + "norm2"].to(dtype), eps)
        layers.append(x)
    h = rms_norm(x, t["final.norm"].to(dtype), eps)
    return h @ t["embed"].to(dtype).T, torch.stack(layers)


def greedy(prompt, steps, t, cfg, dtype=torch.float64):
    """``steps`` tokens after ``prompt``, each the argmax of the last position's logits."""
    toks = list(prompt)
    out = []
    for _ in range(steps):
        logits, _ = forward(toks, t, cfg, dtype)
        out.append(int(torch.argmax(logits[-1])))
        toks.append(out[-1])
    return out
