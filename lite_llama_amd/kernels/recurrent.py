"""Recurrent sequence mixers over ragged steps (csrc/seq_mix.hip): fixed-size fp32 state per (sequence slot, head), carried
from step to step -- the counterpart, for layers without a growing cache, of the attention kernels next door."""

from __future__ import annotations

import torch

from .. import _lib as L


def gated_linear_scan_supported(dk: int, dv: int) -> bool:
    return bool(L.lib().ll_gated_linear_scan_supported(dk, dv))


@torch.no_grad()
def gated_linear_scan(qfv: torch.Tensor, heads: int, dk: int, dv: int, f_bias, lower, norm_weight, eps: float, step,
                      state: torch.Tensor) -> torch.Tensor:
    """HGRN2-style gated linear attention.  ``qfv [n, 2 heads dk + heads dv]`` = the fused projection rows
    ``[q_raw | f_raw | v]``; per head ``f = lower + (1 - lower) sigmoid(f_raw + f_bias)``,
    ``S <- diag(f) S + (1 - f) v^T``, ``o = S^T silu(q_raw)``, then ``o`` RMS-normed over ``dv`` with ``norm_weight``.
    ``state [slots, heads, dk, dv]`` fp32: a sequence whose run starts at position 0 starts from zeros (whatever an earlier
    owner of the slot left), every run leaves its final state.  Returns ``[n, heads dv]`` in the storage dtype."""
    L.require_cuda(qfv, f_bias, lower, norm_weight, state)
    n = qfv.shape[0]
    dt = qfv.dtype
    if qfv.dim() != 2 or qfv.stride(1) != 1 or qfv.shape[1] < 2 * heads * dk + heads * dv:
        raise ValueError("gated_linear_scan: qfv rows hold [q | f | v]")
    if state.dtype != torch.float32 or not state.is_contiguous() or tuple(state.shape[1:]) != (heads, dk, dv):
        raise ValueError("gated_linear_scan: state is contiguous fp32 [slots, heads, dk, dv]")
    for t, size in ((f_bias, heads * dk), (lower, heads * dk), (norm_weight, dv)):
        if t.dtype != dt or t.numel() != size or not t.is_contiguous():
            raise ValueError("gated_linear_scan: gate bias / lower bound [heads dk] and norm weight [dv] in the rows' dtype")
    if step.num_tokens != n:
        raise ValueError("gated_linear_scan: the step describes another number of tokens")
    if not gated_linear_scan_supported(dk, dv):
        raise ValueError(f"gated_linear_scan: head geometry {dk} x {dv} is not served (dv <= 256, <= 128 state rows per thread)")
    out = torch.empty(n, heads * dv, dtype=dt, device=qfv.device)
    # the wide form (a workgroup per 16 state columns; o through an fp32 scratch, then the norm) needs a scratch; the library
    # picks the form (runs of several tokens, or batches too small to fill the chip with a workgroup per (sequence, head))
    scratch = torch.empty(n, heads * dv, dtype=torch.float32, device=qfv.device) if dk <= 256 else None
    es = qfv.element_size()
    base = qfv.data_ptr()
    L.check(L.lib().ll_gated_linear_scan(
        base, base + heads * dk * es, base + 2 * heads * dk * es, qfv.stride(0), f_bias.data_ptr(), lower.data_ptr(),
        norm_weight.data_ptr(), float(eps), out.data_ptr(), step.num_seqs, heads, dk, dv, step.seq_start.data_ptr(),
        step.seq_first_pos.data_ptr(), step.seq_slot.data_ptr(), state.data_ptr(), n, step.longest_run, L.ptr(scratch),
        L.dtype_code(dt), L.stream_ptr()),
        "gated_linear_scan")
    return out


@torch.no_grad()
def mingru_scan(zxg: torch.Tensor, width: int, z_bias, x_bias, step, state: torch.Tensor) -> torch.Tensor:
    """minGRU over a ragged step.  ``zxg [n, >= 3 width]`` = fused projection rows ``[z_raw | x_raw | g_raw]``; per channel
    ``z = sigmoid(z_raw + z_bias)``, ``u = x_raw + x_bias``, candidate ``u + 1/2`` where ``u >= 0`` and ``sigmoid(u)`` below,
    ``S <- (1 - z) S + z candidate``; returns ``S * silu(g_raw)`` ``[n, width]`` in the storage dtype.  ``state
    [slots, width]`` fp32: a sequence whose run starts at position 0 starts from zeros, every run leaves its final state."""
    L.require_cuda(zxg, z_bias, x_bias, state)
    n, dt = zxg.shape[0], zxg.dtype
    if zxg.dim() != 2 or zxg.stride(1) != 1 or zxg.shape[1] < 3 * width:
        raise ValueError("mingru_scan: rows hold [z | x | g]")
    if state.dtype != torch.float32 or not state.is_contiguous() or state.dim() != 2 or state.shape[1] != width:
        raise ValueError("mingru_scan: state is contiguous fp32 [slots, width]")
    for b in (z_bias, x_bias):
        if b is not None and (b.dtype != dt or b.numel() != width or not b.is_contiguous()):
            raise ValueError("mingru_scan: biases are [width] in the rows' dtype")
    if step.num_tokens != n:
        raise ValueError("mingru_scan: the step describes another number of tokens")
    out = torch.empty(n, width, dtype=dt, device=zxg.device)
    es, base = zxg.element_size(), zxg.data_ptr()
    # long runs: chunks of a run are walked side by side (chunk maps, entering states, the chunks again) over an fp32 scratch
    floats = int(L.lib().ll_mingru_scan_scratch_floats(step.num_seqs, width, step.longest_run))
    scratch = torch.empty(floats, dtype=torch.float32, device=zxg.device) if floats else None
    L.check(L.lib().ll_mingru_scan(base, base + width * es, base + 2 * width * es, zxg.stride(0), L.ptr(z_bias), L.ptr(x_bias),
                                   out.data_ptr(), step.num_seqs, width, step.seq_start.data_ptr(), step.seq_first_pos.data_ptr(),
                                   step.seq_slot.data_ptr(), state.data_ptr(), step.longest_run, L.ptr(scratch), L.dtype_code(dt),
                                   L.stream_ptr()), "mingru_scan")
    return out


# ------------------------------------------------------------------------------------- #
# linear attention with a decay (csrc/linear_mix.hip)
# ------------------------------------------------------------------------------------- #
def linear_scan_supported(dk: int, dv: int) -> bool:
    return bool(L.lib().ll_linear_scan_supported(dk, dv))


def _rows(t: torch.Tensor, cols: int, what: str) -> None:
    if t.dim() != 2 or t.stride(1) != 1 or t.shape[1] < cols:
        raise ValueError(f"linear_scan: {what} rows are [n, >= {cols}] with a unit inner stride")


@torch.no_grad()
def linear_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, heads: int, dk: int, dv: int, step, state: torch.Tensor, *,
                qk_heads: int | None = None, act: bool = False, q_scale: float = 1.0, head_decay: torch.Tensor | None = None,
                gate: torch.Tensor | None = None, gate_bias: torch.Tensor | None = None, tau: float = 1.0,
                dt: torch.Tensor | None = None, dt_bias: torch.Tensor | None = None, a_log: torch.Tensor | None = None,
                skip: torch.Tensor | None = None) -> torch.Tensor:
    """Linear attention with a decaying state over a ragged step: per head ``S <- diag(a_t) S + k_t (b_t v_t)^T``,
    ``o_t = S^T q_t (+ skip_h v_t)``.  ``q`` / ``k`` / ``v``: row-strided views ``[n, qk_heads dk]`` / ``[n, heads dv]`` (column
    ranges of a fused projection); ``qk_heads`` (default ``heads``) query / key heads are shared by ``heads / qk_heads``
    neighbouring value heads each.  ``act``: q, k, v pass through silu.  Exactly one decay:

      * ``head_decay [heads]`` fp32: a fixed number per head;
      * ``gate [n, heads dk]`` + ``gate_bias [heads dk]``: ``a = sigmoid(gate + bias)^(1 / tau)`` per key entry;
      * ``dt [n, heads]`` + ``dt_bias``, ``a_log`` (and ``skip``) ``[heads]``: ``dt' = softplus(dt + dt_bias)``,
        ``a = exp(-exp(a_log) dt')``, ``b = dt'``.

    ``state [slots, heads, dk, dv]`` fp32: a sequence whose run starts at position 0 starts from zeros, every run leaves its
    final state.  Decays, step sizes, state and read-out are fp32.  Returns ``o`` fp32 ``[n, heads dv]``."""
    L.require_cuda(q, k, v, state, head_decay, gate, gate_bias, dt, dt_bias, a_log, skip)
    n, st = q.shape[0], q.dtype
    qk_heads = heads if qk_heads is None else qk_heads
    if qk_heads < 1 or heads % qk_heads:
        raise ValueError(f"linear_scan: {heads} value heads do not divide over {qk_heads} query / key heads")
    _rows(q, qk_heads * dk, "query")
    _rows(k, qk_heads * dk, "key")
    _rows(v, heads * dv, "value")
    if k.dtype != st or v.dtype != st or k.shape[0] != n or v.shape[0] != n or step.num_tokens != n:
        raise ValueError("linear_scan: q, k, v of one dtype, one row per token of the step")
    if state.dtype != torch.float32 or not state.is_contiguous() or tuple(state.shape[1:]) != (heads, dk, dv):
        raise ValueError("linear_scan: state is contiguous fp32 [slots, heads, dk, dv]")
    if not linear_scan_supported(dk, dv):
        raise ValueError(f"linear_scan: head geometry {dk} x {dv} is not served (dk <= 256)")
    kinds = [head_decay is not None, gate is not None, dt is not None]
    if sum(kinds) != 1:
        raise ValueError("linear_scan: exactly one of head_decay, gate, dt names the decay")
    kind = kinds.index(True)

    def vec(t, size, what):
        if t is None or t.dtype != st or t.numel() != size or not t.is_contiguous():
            raise ValueError(f"linear_scan: {what} has {size} entries in the rows' dtype")

    if kind == 0 and (head_decay.dtype != torch.float32 or head_decay.numel() != heads or not head_decay.is_contiguous()):
        raise ValueError("linear_scan: head_decay is fp32 [heads]")
    if kind == 1:
        _rows(gate, heads * dk, "decay logit")
        vec(gate_bias, heads * dk, "gate_bias")
        if gate.dtype != st or gate.shape[0] != n or not tau > 0:
            raise ValueError("linear_scan: decay logits in the rows' dtype, one row per token; tau > 0")
    if kind == 2:
        _rows(dt, heads, "step size")
        vec(dt_bias, heads, "dt_bias")
        vec(a_log, heads, "a_log")
        if skip is not None:
            vec(skip, heads, "skip")
        if dt.dtype != st or dt.shape[0] != n:
            raise ValueError("linear_scan: step sizes in the rows' dtype, one row per token")
    o = torch.empty(n, heads * dv, dtype=torch.float32, device=q.device)
    # runs of several tokens: the decays per key entry are evaluated once per token ahead of the scan (its column workgroups
    # would each evaluate them again); decode steps evaluate them in the scan
    pre = torch.empty(n, heads * dk, dtype=torch.float32, device=q.device) if (kind == 1 and step.longest_run != 1 and dv > 16) else None
    L.check(L.lib().ll_linear_scan(
        q.data_ptr(), q.stride(0), k.data_ptr(), k.stride(0), v.data_ptr(), v.stride(0), heads, dk, dv, heads // qk_heads, kind,
        1 if act else 0, float(q_scale), L.ptr(head_decay), L.ptr(gate), gate.stride(0) if gate is not None else 0, L.ptr(gate_bias),
        1.0 / float(tau), L.ptr(dt), dt.stride(0) if dt is not None else 0, L.ptr(dt_bias), L.ptr(a_log), L.ptr(skip), o.data_ptr(),
        step.num_seqs, step.seq_start.data_ptr(), step.seq_first_pos.data_ptr(), step.seq_slot.data_ptr(), state.data_ptr(),
        L.ptr(pre), n, int(step.longest_run), L.dtype_code(st), L.stream_ptr()), "linear_scan")
    return o


_GATES = {None: 0, "silu": 1, "sigmoid": 2}


@torch.no_grad()
def gated_out_norm(o: torch.Tensor, weight: torch.Tensor | None, eps: float, *, parts: int = 1, gate: torch.Tensor | None = None,
                   gate_kind: str | None = None, gate_first: bool = False, scale: float = 1.0, out: torch.Tensor | None = None,
                   dtype=None) -> torch.Tensor:
    """A recurrence's read-out ``o`` (fp32 ``[n, width]``) -> RMS norm over ``parts`` equal consecutive parts of the row (each
    divided by ``sqrt(mean(part^2) + eps)``), times ``weight`` -- ``[width]``, or a shorter vector repeated along the row (one
    weight vector shared by all heads) --, times ``silu`` / ``sigmoid`` of ``gate [n, width]`` (a row-strided view) either after
    the norm or, with ``gate_first``, before it; times ``scale``.  fp32 until the one rounding to the storage dtype.  ``out``: a
    ``[n, width]`` view with a unit inner stride (a column range of the next projection's input)."""
    L.require_cuda(o, weight, gate, out)
    n, width = o.shape
    dt = dtype or (weight.dtype if weight is not None else gate.dtype)
    if o.dtype != torch.float32 or not o.is_contiguous() or width % parts:
        raise ValueError("gated_out_norm: a contiguous fp32 read-out whose width the parts divide")
    if weight is not None and (weight.dtype != dt or not weight.is_contiguous() or width % weight.numel()):
        raise ValueError("gated_out_norm: the weight's length divides the width, in the storage dtype")
    if (gate is None) != (gate_kind is None):
        raise ValueError("gated_out_norm: a gate comes with its kind")
    if gate is not None and (gate.dtype != dt or gate.dim() != 2 or gate.shape[0] != n or gate.shape[1] < width or gate.stride(1) != 1):
        raise ValueError("gated_out_norm: gate rows are [n, >= width] in the storage dtype with a unit inner stride")
    if out is None:
        out = torch.empty(n, width, dtype=dt, device=o.device)
    elif out.dtype != dt or tuple(out.shape) != (n, width) or out.stride(1) != 1:
        raise ValueError("gated_out_norm: out is [n, width] in the storage dtype with a unit inner stride")
    L.check(L.lib().ll_gated_out_norm(out.data_ptr(), max(out.stride(0), width), o.data_ptr(), L.ptr(gate),
                                      max(gate.stride(0), width) if gate is not None else 0, _GATES[gate_kind], 1 if gate_first else 0,
                                      L.ptr(weight), weight.numel() if weight is not None else 0, float(eps), float(scale), n, width,
                                      int(parts), L.dtype_code(dt), L.stream_ptr()), "gated_out_norm")
    return out


@torch.no_grad()
def conv_act(rows: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None, step, state: torch.Tensor | None) -> torch.Tensor:
    """``silu(bias + causal convolution)`` per channel over a ragged step: ``rows [n, channels]`` (a row-strided view),
    ``weight [channels, taps]`` (the last column is the current token's; zeros in front of position 0).  ``state
    [2, slots, taps - 1, channels]`` in the rows' dtype carries the raw rows of a sequence's last positions (the half named by
    the sequence's parity is read, the other written).  fp32 sums; returns ``[n, channels]`` in the rows' dtype."""
    L.require_cuda(rows, weight, bias, state)
    n, dt = rows.shape[0], rows.dtype
    channels, taps = weight.shape
    if rows.dim() != 2 or rows.stride(1) != 1 or rows.shape[1] < channels or step.num_tokens != n:
        raise ValueError("conv_act: rows hold the channels of the step's tokens")
    if weight.dtype != dt or not weight.is_contiguous() or (bias is not None and (bias.dtype != dt or bias.numel() != channels
                                                                                  or not bias.is_contiguous())):
        raise ValueError("conv_act: weights [channels, taps] and a bias per channel in the rows' dtype")
    if taps > 1 and (state is None or state.dtype != dt or state.dim() != 4 or state.shape[0] != 2
                     or tuple(state.shape[2:]) != (taps - 1, channels) or not state.is_contiguous()):
        raise ValueError("conv_act: the carried rows are [2, slots, taps - 1, channels] in the rows' dtype")
    out = torch.empty(n, channels, dtype=dt, device=rows.device)
    L.check(L.lib().ll_conv_act(out.data_ptr(), channels, rows.data_ptr(), max(rows.stride(0), channels), weight.data_ptr(), L.ptr(bias),
                                channels, taps, L.ptr(state) if taps > 1 else 0, state[0].numel() if taps > 1 else 0,
                                step.tok_seq.data_ptr(), step.tok_pos.data_ptr(), step.seq_start.data_ptr(),
                                step.seq_first_pos.data_ptr(), step.seq_slot.data_ptr(), step.seq_parity.data_ptr(), n,
                                L.dtype_code(dt), L.stream_ptr()), "conv_act")
    return out
