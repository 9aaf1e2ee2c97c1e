"""flash_decoding / flash_attention2_no_pad -- mirror of lite_llama/kernels/flashdecoding.py:316-380
and flashattention2_nopad.py:175-231 over the HIP C-ABI."""

from __future__ import annotations

import os

import torch

from .. import _lib as L


# zeroed, self-cleaning counters for the one-launch merge (kernels never allocate; grown outside graph
# capture; outgrown vectors stay alive for graphs that captured their address).  One vector per
# (device, stream) for eager calls, one per device for captures -- see _lib.scratch_keys.
_fd_counters: dict = {}
_fd_keepalive: list = []


def _grow_counters(key, device, entries: int):
    cur = _fd_counters.get(key)
    if cur is not None and cur.numel() >= entries:
        return cur
    if torch.cuda.is_current_stream_capturing():
        return None  # first use inside a capture: take the two-launch form this once
    if cur is not None:
        _fd_keepalive.append(cur)
    cur = torch.zeros(max(entries, 4096), dtype=torch.int32, device=device)
    _fd_counters[key] = cur
    return cur


def _merge_counters(device, entries: int):
    key, cap = L.scratch_keys(device)
    if key != cap:
        _grow_counters(cap, device, entries)
    return _grow_counters(key, device, entries)


@torch.no_grad()
def flash_decoding(
    q,
    k_cache,
    v_cache,
    qk_scale,
    b_req_tokens_table,
    b_req_idx,
    b_seq_len,
    max_actual_seq_len,
):
    """Decode attention for one new token per batch row against the token-attention pool.

    ``k_cache`` / ``v_cache`` may be strided views of ``[max_tokens, 2*Hkv, D]`` (last dim
    contiguous); index tensors may be int32 or int64; the output is a fresh ``[B, Hq, D]``.
    Scratch (``mid_o``, ``mid_o_logexpsum``) is allocated per call like the reference does
    (flashdecoding.py:347-358) -- from torch's caching allocator, so it is graph-safe.
    """
    L.require_cuda(q, k_cache, v_cache, b_req_tokens_table, b_req_idx, b_seq_len)
    assert q.shape[-1] == k_cache.shape[-1] == v_cache.shape[-1]
    assert b_req_tokens_table.dtype == torch.int32
    batchs, num_heads, head_dim = q.shape
    if q.stride(-1) != 1:
        q = q.contiguous()
    assert k_cache.stride(-1) == 1 and v_cache.stride(-1) == 1
    if b_req_tokens_table.stride(1) != 1:
        b_req_tokens_table = b_req_tokens_table.contiguous()
    max_len = int(max_actual_seq_len)
    nparts = L.lib().ll_flash_decoding_num_partitions(max_len)
    mid_o = torch.empty((batchs, num_heads, max(nparts, 1), head_dim), dtype=torch.float32, device=q.device)
    out = torch.empty_like(q, memory_format=torch.contiguous_format)
    n_kv = k_cache.shape[1]
    counters = _merge_counters(q.device, batchs * n_kv * ((num_heads // n_kv + 15) // 16))
    # one-launch form: a cache line (32 floats) per log-sum-exp record
    mid_lse = torch.empty((batchs, num_heads, max(nparts, 1), 1 if counters is None else 32), dtype=torch.float32,
                          device=q.device)
    L.check(
        L.lib().ll_flash_decoding(
            out.data_ptr(), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
            b_req_tokens_table.data_ptr(), b_req_idx.data_ptr(), b_seq_len.data_ptr(),
            mid_o.data_ptr(), mid_lse.data_ptr(), batchs, num_heads, k_cache.shape[1], head_dim,
            max_len, float(qk_scale), q.stride(0), q.stride(1), k_cache.stride(0), k_cache.stride(1),
            v_cache.stride(0), v_cache.stride(1), out.stride(0), out.stride(1),
            b_req_tokens_table.stride(0), L.dtype_code(q.dtype), L.index_width(b_req_idx),
            L.index_width(b_seq_len), L.ptr(counters), L.stream_ptr(),
        ),
        "flash_decoding",
    )
    return out


@torch.no_grad()
def flash_decoding_fp8kv(q, k_cache, v_cache, qk_scale, b_req_tokens_table, b_req_idx, b_seq_len, max_actual_seq_len,
                         k_scale: float = 1.0, v_scale: float = 1.0):
    """``flash_decoding`` over an fp8 (OCP e4m3) pool written by ``update_kv_buffer_fp8`` (extension): ``k_cache`` /
    ``v_cache`` are uint8 / float8_e4m3fn views ``[rows, Hkv, D]``; fp16 queries, ``D`` 64 or 128."""
    L.require_cuda(q, k_cache, v_cache, b_req_tokens_table, b_req_idx, b_seq_len)
    assert q.dtype == torch.float16 and k_cache.element_size() == 1 and v_cache.element_size() == 1
    assert q.shape[-1] == k_cache.shape[-1] == v_cache.shape[-1] and b_req_tokens_table.dtype == torch.int32
    batchs, num_heads, head_dim = q.shape
    if q.stride(-1) != 1:
        q = q.contiguous()
    assert k_cache.stride(-1) == 1 and v_cache.stride(-1) == 1
    if b_req_tokens_table.stride(1) != 1:
        b_req_tokens_table = b_req_tokens_table.contiguous()
    max_len = int(max_actual_seq_len)
    nparts = L.lib().ll_flash_decoding_num_partitions(max_len)
    mid_o = torch.empty((batchs, num_heads, max(nparts, 1), head_dim), dtype=torch.float32, device=q.device)
    out = torch.empty_like(q, memory_format=torch.contiguous_format)
    n_kv = k_cache.shape[1]
    counters = _merge_counters(q.device, batchs * n_kv * ((num_heads // n_kv + 15) // 16))
    if counters is None:
        raise L.KernelError("flash_decoding_fp8kv needs the merge counters (not available during this capture)")
    mid_lse = torch.empty((batchs, num_heads, max(nparts, 1), 32), dtype=torch.float32, device=q.device)
    L.check(
        L.lib().ll_flash_decoding_fp8kv(
            out.data_ptr(), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), b_req_tokens_table.data_ptr(),
            b_req_idx.data_ptr(), b_seq_len.data_ptr(), mid_o.data_ptr(), mid_lse.data_ptr(), batchs, num_heads, n_kv,
            head_dim, max_len, float(qk_scale), float(k_scale), float(v_scale), q.stride(0), q.stride(1),
            k_cache.stride(0), k_cache.stride(1), v_cache.stride(0), v_cache.stride(1), out.stride(0), out.stride(1),
            b_req_tokens_table.stride(0), L.index_width(b_req_idx), L.index_width(b_seq_len), L.ptr(counters),
            L.stream_ptr(),
        ),
        "flash_decoding_fp8kv",
    )
    return out


def decode_attention_supported(q, kv, cos, n_kv_heads: int) -> bool:
    """Shapes the one-launch decode attention serves: head_dim >= 64, at most 16 query heads per KV
    head, dense [heads, head_dim] rows, 16-bit tables of the activation dtype."""
    n, hq, hd = q.shape
    return (hd >= 64 and hd % 32 == 0 and hq % n_kv_heads == 0 and hq // n_kv_heads <= 16 and q.stride(2) == 1
            and q.stride(1) == hd and kv.stride(2) == 1 and kv.stride(1) == hd and cos.dtype == q.dtype
            and q.dtype in (torch.float16, torch.bfloat16) and q.stride(0) % 8 == 0 and kv.stride(0) % 8 == 0)


@torch.no_grad()
def _head_norm_ok(qk_norm, head_dim: int, dtype) -> bool:
    if qk_norm is None:
        return True
    qw, kw, _ = qk_norm
    return (head_dim == 128 and all(w.dtype == dtype and w.is_contiguous() and w.numel() == head_dim and w.is_cuda
                                    for w in (qw, kw)))


@torch.no_grad()
def decode_attention(q, kv, cos_table, sin_table, positions, select_index, kv_buffer, qk_scale, b_req_tokens_table,
                     b_req_idx, b_seq_len, max_actual_seq_len, qk_norm=None):
    """Extension: ``rope_and_cache(q, kv, tables, positions)`` + ``flash_decoding(...)`` in ONE launch
    (same values).  ``q [B, Hq, D]`` un-rotated (left untouched), ``kv [B, 2*Hkv, D]`` this step's K
    heads then V heads (left untouched), ``kv_buffer [max_tokens, 2*Hkv, D]`` the layer's pool: row
    ``select_index[b]`` receives the rotated K and the V.  ``qk_norm = (q_weight, k_weight, eps)`` (Qwen3, head_dim 128):
    the per-head RMSNorm of q and of the new K heads runs inside the launch, in front of the rotation, with the values
    of ``skip_rmsnorm`` on the ``[.., D]`` views.  Returns ``None`` when the shape is not
    served or the merge counters cannot be set up (caller runs the two-call form)."""
    L.require_cuda(q, kv, cos_table, sin_table, positions, select_index, kv_buffer, b_req_tokens_table, b_req_idx,
                   b_seq_len)
    batchs, num_heads, head_dim = q.shape
    n_kv = kv.shape[1] // 2
    if not decode_attention_supported(q, kv, cos_table, n_kv) or not _head_norm_ok(qk_norm, head_dim, q.dtype):
        return None
    counters = _merge_counters(q.device, batchs * n_kv)
    positions = positions.reshape(-1)
    if (counters is None or sin_table.dtype != cos_table.dtype or cos_table.dim() != 2 or cos_table.stride(1) != 1
            or sin_table.stride(1) != 1 or cos_table.stride(0) != sin_table.stride(0) or cos_table.stride(0) % 8 != 0
            or positions.dtype != torch.int64 or not positions.is_contiguous() or positions.shape[0] != batchs
            or kv_buffer.stride(2) != 1 or b_req_tokens_table.dtype != torch.int32 or b_req_tokens_table.stride(1) != 1):
        return None
    k_cache, v_cache = kv_buffer[:, :n_kv], kv_buffer[:, n_kv:]
    max_len = int(max_actual_seq_len)
    nparts = L.lib().ll_flash_decoding_num_partitions(max_len)
    mid_o = torch.empty((batchs, num_heads, max(nparts, 1), head_dim), dtype=torch.float32, device=q.device)
    mid_lse = torch.empty((batchs, num_heads, max(nparts, 1), 32), dtype=torch.float32, device=q.device)
    out = torch.empty((batchs, num_heads, head_dim), dtype=q.dtype, device=q.device)
    L.check(
        L.lib().ll_decode_attention(
            out.data_ptr(), q.data_ptr(), kv.data_ptr(), kv.stride(0), cos_table.data_ptr(), sin_table.data_ptr(),
            cos_table.stride(0), positions.data_ptr(), select_index.data_ptr(), L.index_width(select_index),
            k_cache.data_ptr(), v_cache.data_ptr(), b_req_tokens_table.data_ptr(), b_req_idx.data_ptr(),
            b_seq_len.data_ptr(), mid_o.data_ptr(), mid_lse.data_ptr(), batchs, num_heads, n_kv, head_dim, max_len,
            float(qk_scale), q.stride(0), q.stride(1), k_cache.stride(0), k_cache.stride(1), v_cache.stride(0),
            v_cache.stride(1), out.stride(0), out.stride(1), b_req_tokens_table.stride(0), L.dtype_code(q.dtype),
            L.index_width(b_req_idx), L.index_width(b_seq_len), counters.data_ptr(),
            L.ptr(None if qk_norm is None else qk_norm[0]), L.ptr(None if qk_norm is None else qk_norm[1]),
            0.0 if qk_norm is None else float(qk_norm[2]), L.stream_ptr(),
        ),
        "decode_attention",
    )
    return out


def decode_attention_partials_supported(max_actual_seq_len, num_heads: int, num_kv_heads: int, head_dim: int, batch: int = 1) -> bool:
    """Whether :func:`decode_attention_partials` serves this step (known before the projection is launched): the
    one-workgroup-per-(row, KV head) form -- contexts of 129 .. 1024 tokens at any batch, longer ones (round 6: the waves walk the
    partitions) when ``batch x KV heads`` alone fills half the chip."""
    waves = L.lib().ll_flash_decoding_group_waves(int(max_actual_seq_len), int(batch) * int(num_kv_heads))
    return (waves >= 2 and head_dim >= 64 and head_dim % 32 == 0 and num_heads % num_kv_heads == 0
            and num_heads // num_kv_heads <= 16 and (num_heads // num_kv_heads + 2) * head_dim // 4 <= 128 * waves)


@torch.no_grad()
def decode_attention_partials(parts, bias, num_heads: int, num_kv_heads: int, head_dim: int, cos_table, sin_table,
                              positions, select_index, kv_buffer, qk_scale, b_req_tokens_table, b_req_idx, b_seq_len,
                              max_actual_seq_len, qk_norm=None):
    """:func:`decode_attention` whose ``q | k | v`` come as the fp32 split-K partials of the fused projection
    (``PartialSums`` ``[S, B, (Hq + 2 Hkv) D]``, ``bias`` the projection bias or ``None``): every workgroup adds the
    partials of its (row, KV head) -- plus bias, one rounding to the pool dtype: the value the projection itself would
    have stored -- and continues as ``decode_attention`` (``qk_norm`` as there).  ``parts`` may also be the
    ``ScaledInt32Partials`` of a smoothquant projection (fp16, head_dim 128): the launch applies the scale epilogue.  Returns ``None`` when the shape is not served (contexts of
    129..1024 tokens -- any longer one when batch x KV heads >= 128 workgroups --, head_dim >= 64, <= 16 query heads per KV head):
    finish the sums and call ``decode_attention``."""
    p = parts.parts
    scaled = p.dtype == torch.int32  # smoothquant: exact int32 planes + per-token / per-channel scales (ScaledInt32Partials)
    if scaled and (qk_norm is not None or head_dim != 128 or kv_buffer.dtype != torch.float16
                   or getattr(parts, "a_scale", None) is None):
        return None
    L.require_cuda(p, bias, cos_table, sin_table, positions, select_index, kv_buffer, b_req_tokens_table, b_req_idx, b_seq_len)
    s_count, batchs, row_w = p.shape
    dt = kv_buffer.dtype
    positions = positions.reshape(-1)
    if ((p.dtype != torch.float32 and not scaled) or row_w != (num_heads + 2 * num_kv_heads) * head_dim or head_dim < 64 or head_dim % 32 or num_heads % num_kv_heads
            or num_heads // num_kv_heads > 16 or s_count > 8 or not p.is_contiguous() or parts.dtype != dt
            or dt not in (torch.float16, torch.bfloat16) or cos_table.dtype != dt or sin_table.dtype != dt
            or cos_table.dim() != 2 or cos_table.stride(1) != 1 or sin_table.stride(1) != 1
            or cos_table.stride(0) != sin_table.stride(0) or cos_table.stride(0) % 8 != 0
            or positions.dtype != torch.int64 or not positions.is_contiguous() or positions.shape[0] != batchs
            or kv_buffer.stride(2) != 1 or b_req_tokens_table.dtype != torch.int32 or b_req_tokens_table.stride(1) != 1
            or (bias is not None and (bias.dtype != dt or not bias.is_contiguous() or bias.numel() != row_w))
            or not _head_norm_ok(qk_norm, head_dim, dt)):
        return None
    max_len = int(max_actual_seq_len)
    waves = L.lib().ll_flash_decoding_group_waves(max_len, batchs * num_kv_heads)  # the one-workgroup form (0: not applicable)
    if waves < 2 or (num_heads // num_kv_heads + 2) * head_dim // 4 > 128 * waves:
        return None
    k_cache, v_cache = kv_buffer[:, :num_kv_heads], kv_buffer[:, num_kv_heads:]
    out = torch.empty((batchs, num_heads, head_dim), dtype=dt, device=p.device)
    L.check(
        L.lib().ll_decode_attention_partials(
            out.data_ptr(), p.data_ptr(), s_count, L.ptr(bias), cos_table.data_ptr(), sin_table.data_ptr(),
            cos_table.stride(0), positions.data_ptr(), select_index.data_ptr(), L.index_width(select_index),
            k_cache.data_ptr(), v_cache.data_ptr(), b_req_tokens_table.data_ptr(), b_req_idx.data_ptr(),
            b_seq_len.data_ptr(), batchs, num_heads, num_kv_heads, head_dim, max_len, float(qk_scale),
            k_cache.stride(0), k_cache.stride(1), v_cache.stride(0), v_cache.stride(1), out.stride(0), out.stride(1),
            b_req_tokens_table.stride(0), L.dtype_code(dt), L.index_width(b_req_idx), L.index_width(b_seq_len),
            L.ptr(None if qk_norm is None else qk_norm[0]), L.ptr(None if qk_norm is None else qk_norm[1]),
            0.0 if qk_norm is None else float(qk_norm[2]), parts.a_scale.data_ptr() if scaled else 0,
            parts.w_scale.data_ptr() if scaled else 0, L.stream_ptr(),
        ),
        "decode_attention_partials",
    )
    return out


@torch.no_grad()
def flash_attention2_no_pad(q, k, v, sm_scale, b_start_loc, b_seq_len, max_seq_len):
    """Varlen causal prefill attention (``sm_scale`` must already include log2(e); the
    kernel evaluates exp2).  fp32 inputs are cast to fp16 like the reference's
    ``custom_fwd(cast_inputs=torch.float16)``."""
    L.require_cuda(q, k, v, b_start_loc, b_seq_len)
    if q.dtype == torch.float32:
        q, k, v = q.half(), k.half(), v.half()
    if q.stride(-1) != 1:
        q = q.contiguous()
    if k.stride(-1) != 1:
        k = k.contiguous()
    if v.stride(-1) != 1:
        v = v.contiguous()
    output = torch.empty_like(q, memory_format=torch.contiguous_format)
    batchs = b_seq_len.shape[0]
    n_heads, head_dim = q.shape[1], q.shape[2]
    L.check(
        L.lib().ll_flash_attention_nopad(
            output.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), b_start_loc.data_ptr(),
            b_seq_len.data_ptr(), batchs, n_heads, k.shape[1], head_dim, int(max_seq_len),
            float(sm_scale), q.stride(0), q.stride(1), k.stride(0), k.stride(1), v.stride(0),
            v.stride(1), output.stride(0), output.stride(1), L.dtype_code(q.dtype),
            L.index_width(b_start_loc), L.index_width(b_seq_len), L.stream_ptr(),
        ),
        "flash_attention2_no_pad",
    )
    return output


# ------------------------------------------------------------------------------------- #
# ragged steps against a paged cache with separate key / value widths (csrc/ragged_attn.hip)
# ------------------------------------------------------------------------------------- #
@torch.no_grad()
def qk_norm_cache(qkv, heads: int, kv_heads: int, dk: int, dv: int, q_weight, k_weight, eps: float, temp_coef: float,
                  temp_every: int, step, k_cache, v_cache):
    """Fused projection rows ``[q | k | v]`` -> queries ``[n, heads, dk]`` (per-head RMS norm, then the position temperature
    ``1 + temp_coef ln(floor((pos + 1) / temp_every) + 1)``); normed keys and values land in the cache rows ``step.select``."""
    L.require_cuda(qkv, k_cache, v_cache)
    n, dt = qkv.shape[0], qkv.dtype
    if qkv.dim() != 2 or qkv.stride(1) != 1 or qkv.shape[1] < (heads + kv_heads) * dk + kv_heads * dv:
        raise ValueError("qk_norm_cache: rows hold [q | k | v]")
    if k_cache.dtype != dt or v_cache.dtype != dt or tuple(k_cache.shape[1:]) != (kv_heads, dk) \
            or tuple(v_cache.shape[1:]) != (kv_heads, dv) or not (k_cache.is_contiguous() and v_cache.is_contiguous()):
        raise ValueError("qk_norm_cache: caches are contiguous [rows, kv_heads, dk] / [rows, kv_heads, dv] in the rows' dtype")
    for w in (q_weight, k_weight):
        if w is not None and (w.dtype != dt or w.numel() != dk or not w.is_contiguous()):
            raise ValueError("qk_norm_cache: norm weights are [dk] in the rows' dtype")
    if step.num_tokens != n:
        raise ValueError("qk_norm_cache: the step describes another number of tokens")
    q = torch.empty(n, heads, dk, dtype=dt, device=qkv.device)
    L.check(L.lib().ll_qk_norm_cache(qkv.data_ptr(), qkv.stride(0), L.ptr(q_weight), L.ptr(k_weight), float(eps), float(temp_coef),
                                     int(temp_every), step.tok_pos.data_ptr(), step.select.data_ptr(), q.data_ptr(),
                                     k_cache.data_ptr(), v_cache.data_ptr(), n, heads, kv_heads, dk, dv, L.dtype_code(dt),
                                     L.stream_ptr()), "qk_norm_cache")
    return q


@torch.no_grad()
def rotation_table(step, freq, pairs: int, amp: float = 1.0):
    """fp32 ``[n, 2 * pairs4]`` (``pairs4``: ``pairs`` rounded up to a multiple of 4, the padding zero): per token of the step and
    entry pair ``(cos(position * freq[i]) * amp, sin(position * freq[i]) * amp)``."""
    L.require_cuda(freq)
    if freq.dtype != torch.float32 or freq.numel() < pairs or not freq.is_contiguous() or pairs < 1:
        raise ValueError("rotation_table: fp32 frequencies, one per rotated pair")
    out = torch.empty(step.num_tokens, 2 * (-(-pairs // 4) * 4), dtype=torch.float32, device=freq.device)
    L.check(L.lib().ll_rotation_table(step.tok_pos.data_ptr(), freq.data_ptr(), int(pairs), float(amp), out.data_ptr(), step.num_tokens,
                                      L.stream_ptr()), "rotation_table")
    return out


@torch.no_grad()
def conv_rope_cache(qkv, heads: int, kv_heads: int, dk: int, dv: int, step, k_cache, v_cache, *, bias=None, conv_weight=None,
                    conv_state=None, freq=None, pairs: int = 0, amp: float = 1.0, unit_norm: bool = False, eps: float = 0.0,
                    v_source=None, v_blend=None, rot_table=None):
    """Fused projection rows ``[q | k | v]`` -> queries ``[n, heads, dk]``; keys and values land in the cache rows
    ``step.select``.  Channel by channel, in fp32: ``+ bias``; a causal convolution over the sequence's positions with
    ``conv_weight [channels, taps]`` (``y_t = sum_j w[:, j] u_(t - taps + 1 + j)``, zeros in front of position 0), the raw rows of
    a sequence's last ``taps - 1`` positions carried in ``conv_state [2, slots, taps - 1, channels]`` (the half named by the
    sequence's parity is read, the other written); entry pairs ``(2i, 2i + 1)``, ``i < pairs``, of every q / k head rotated by
    ``position * freq[i]`` with cos / sin times ``amp``; q / k heads divided by ``sqrt(mean + eps)`` when ``unit_norm``; values
    become ``(1 - b) v + b v_source[select]`` when ``v_source [rows, kv_heads, dv]`` (another layer's value cache) and the
    one-element tensor ``v_blend`` are given.  ``rot_table``: :func:`rotation_table` of this step for these frequencies (made
    here when absent; layers that rotate alike share one)."""
    L.require_cuda(qkv, k_cache, v_cache, bias, conv_weight, conv_state, freq, v_source, v_blend)
    n, dt = qkv.shape[0], qkv.dtype
    channels = (heads + kv_heads) * dk + kv_heads * dv
    if qkv.dim() != 2 or qkv.stride(1) != 1 or qkv.shape[1] < channels or step.num_tokens != n:
        raise ValueError("conv_rope_cache: rows hold [q | k | v] of the step's tokens")
    if k_cache.dtype != dt or v_cache.dtype != dt or tuple(k_cache.shape[1:]) != (kv_heads, dk) \
            or tuple(v_cache.shape[1:]) != (kv_heads, dv) or not (k_cache.is_contiguous() and v_cache.is_contiguous()):
        raise ValueError("conv_rope_cache: caches are contiguous [rows, kv_heads, dk] / [rows, kv_heads, dv] in the rows' dtype")
    if bias is not None and (bias.dtype != dt or bias.numel() != channels or not bias.is_contiguous()):
        raise ValueError("conv_rope_cache: one bias per channel, in the rows' dtype")
    taps = 0
    if conv_weight is not None:
        if conv_weight.dtype != dt or conv_weight.dim() != 2 or conv_weight.shape[0] != channels or not conv_weight.is_contiguous():
            raise ValueError("conv_rope_cache: convolution weights are [channels, taps] in the rows' dtype")
        taps = conv_weight.shape[1]
        if taps > 1 and (conv_state is None or conv_state.dtype != dt or conv_state.dim() != 4 or conv_state.shape[0] != 2
                         or tuple(conv_state.shape[2:]) != (taps - 1, channels) or not conv_state.is_contiguous()):
            raise ValueError("conv_rope_cache: the carried rows are [2, slots, taps - 1, channels] in the rows' dtype")
    if pairs and (freq is None or freq.dtype != torch.float32 or freq.numel() < pairs or not freq.is_contiguous() or 2 * pairs > dk):
        raise ValueError("conv_rope_cache: fp32 frequencies, one per rotated pair of a head")
    if v_source is not None and (v_blend is None or v_blend.dtype != dt or v_blend.numel() != 1 or v_source.dtype != dt
                                 or tuple(v_source.shape[1:]) != (kv_heads, dv) or not v_source.is_contiguous()
                                 or v_source.shape[0] != v_cache.shape[0]):
        raise ValueError("conv_rope_cache: the blended values are another cache of this one's shape, with a one-element weight")
    if pairs and rot_table is None:
        rot_table = rotation_table(step, freq, pairs, amp)
    if pairs and (rot_table.dtype != torch.float32 or tuple(rot_table.shape) != (n, 2 * (-(-pairs // 4) * 4))
                  or not rot_table.is_contiguous()):
        raise ValueError("conv_rope_cache: the rotation table is what rotation_table() returns for this step and these pairs")
    q = torch.empty(n, heads, dk, dtype=dt, device=qkv.device)
    half = conv_state[0].numel() if (conv_state is not None and taps > 1) else 0
    L.check(L.lib().ll_conv_rope_cache(
        qkv.data_ptr(), qkv.stride(0), L.ptr(bias), L.ptr(conv_weight), taps, L.ptr(conv_state) if taps > 1 else 0, half,
        L.ptr(freq) if pairs else 0, int(pairs), float(amp), L.ptr(rot_table) if pairs else 0, 1 if unit_norm else 0, float(eps),
        L.ptr(v_source),
        v_source.stride(0) if v_source is not None else 0, L.ptr(v_blend) if v_source is not None else 0, step.tok_seq.data_ptr(),
        step.tok_pos.data_ptr(), step.select.data_ptr(), step.seq_start.data_ptr(), step.seq_first_pos.data_ptr(),
        step.seq_slot.data_ptr(), step.seq_parity.data_ptr(), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), n, heads,
        kv_heads, dk, dv, L.dtype_code(dt), L.stream_ptr()), "conv_rope_cache")
    return q


@torch.no_grad()
def rownorm_rope_cache(qkv, heads: int, kv_heads: int, dk: int, dv: int, step, k_cache, v_cache, *, q_weight=None, k_weight=None,
                       eps: float = 0.0, freq=None, pairs: int = 0, value_scale: float = 1.0):
    """Fused projection rows ``[q | k | v]`` -> queries ``[n, heads, dk]``; keys and values land in the cache rows
    ``step.select``.  ``q_weight [heads dk]`` / ``k_weight [kv_heads dk]``: RMS norm over the WHOLE q (k) row -- one mean over
    all heads' entries -- times a weight per entry (``None``: no norm).  Then entry ``i < pairs`` of every q / k head is rotated
    with entry ``i + pairs`` by ``position * freq[i]``: ``(u, w) -> (u cos - w sin, w cos + u sin)``; entries from ``2 pairs`` on
    pass unchanged.  Values enter the cache times ``value_scale`` (a constant factor of the attention's result, applied where
    it costs nothing).  Norms, angles and the rotation are fp32."""
    L.require_cuda(qkv, k_cache, v_cache, q_weight, k_weight, freq)
    n, dt = qkv.shape[0], qkv.dtype
    if qkv.dim() != 2 or qkv.stride(1) != 1 or qkv.shape[1] < (heads + kv_heads) * dk + kv_heads * dv or step.num_tokens != n:
        raise ValueError("rownorm_rope_cache: rows hold [q | k | v] of the step's tokens")
    if k_cache.dtype != dt or v_cache.dtype != dt or tuple(k_cache.shape[1:]) != (kv_heads, dk) \
            or tuple(v_cache.shape[1:]) != (kv_heads, dv) or not (k_cache.is_contiguous() and v_cache.is_contiguous()):
        raise ValueError("rownorm_rope_cache: caches are contiguous [rows, kv_heads, dk] / [rows, kv_heads, dv] in the rows' dtype")
    for w, size in ((q_weight, heads * dk), (k_weight, kv_heads * dk)):
        if w is not None and (w.dtype != dt or w.numel() != size or not w.is_contiguous()):
            raise ValueError("rownorm_rope_cache: norm weights hold one entry per entry of the q / k row, in the rows' dtype")
    if pairs and (freq is None or freq.dtype != torch.float32 or freq.numel() < pairs or not freq.is_contiguous() or 2 * pairs > dk):
        raise ValueError("rownorm_rope_cache: fp32 frequencies, one per rotated pair of a head")
    q = torch.empty(n, heads, dk, dtype=dt, device=qkv.device)
    L.check(L.lib().ll_rownorm_rope_cache(qkv.data_ptr(), max(qkv.stride(0), qkv.shape[1]) if n <= 1 else qkv.stride(0), L.ptr(q_weight),
                                          L.ptr(k_weight), float(eps), L.ptr(freq) if pairs else 0, int(pairs), float(value_scale),
                                          step.tok_pos.data_ptr(), step.select.data_ptr(), q.data_ptr(), k_cache.data_ptr(),
                                          v_cache.data_ptr(), n, heads, kv_heads, dk, dv, L.dtype_code(dt), L.stream_ptr()),
            "rownorm_rope_cache")
    return q


@torch.no_grad()
def ragged_attention(q, k_cache, v_cache, scale: float, step, token_table, sink=None, window: int = 0, keep_first: int = 0,
                     out=None):
    """Causal softmax attention of every token of a ragged step against positions ``0 .. its own`` of its sequence, keys and
    values read through ``token_table[request][position]``; ``sink [heads]`` adds ``exp(sink_h)`` to each head's denominator;
    ``window > 0`` keeps the last ``window`` positions (the token's own included) and, besides them, the sequence's first
    ``keep_first`` positions.  ``k_cache [rows, kv_heads, dk]`` /
    ``v_cache [rows, kv_heads, dv]`` may be row-strided views (the values of a latent cache are a column range of its key
    rows).  Scores, weights and the output sum are fp32.  Returns ``[n, heads * dv]`` (``out``: a view of that shape with a
    unit inner stride, e.g. a column range of the next projection's input)."""
    L.require_cuda(q, k_cache, v_cache, token_table)
    n, heads, dk = q.shape
    kv_heads, dv = v_cache.shape[1], v_cache.shape[2]
    dt = q.dtype
    if not q.is_contiguous() or k_cache.dtype != dt or v_cache.dtype != dt or k_cache.shape[1:] != (kv_heads, dk):
        raise ValueError("ragged_attention: q [n, heads, dk], caches [rows, kv_heads, dk] / [rows, kv_heads, dv], one dtype")
    for c, w in ((k_cache, dk), (v_cache, dv)):
        if c.stride(2) != 1 or (kv_heads > 1 and c.stride(1) != w) or c.stride(0) < kv_heads * w:
            raise ValueError("ragged_attention: cache rows hold their heads densely (only the row stride is free)")
    if token_table.dtype != torch.int32 or token_table.stride(1) != 1:
        raise ValueError("ragged_attention: the token table is row-major int32")
    if sink is not None and (sink.dtype != dt or sink.numel() != heads or not sink.is_contiguous()):
        raise ValueError("ragged_attention: sink is [heads] in the queries' dtype")
    if step.num_tokens != n:
        raise ValueError("ragged_attention: the step describes another number of tokens")
    ks, vs = k_cache.stride(0), v_cache.stride(0)
    if out is None:
        out = torch.empty(n, heads * dv, dtype=dt, device=q.device)
    elif out.dtype != dt or tuple(out.shape) != (n, heads * dv) or out.stride(1) != 1 or not out.is_cuda:
        raise ValueError("ragged_attention: out is [n, heads * dv] in the queries' dtype with a unit inner stride")
    os_ = max(out.stride(0), heads * dv) if n <= 1 else out.stride(0)
    if window <= 0:
        keep_first = 0
    if (step.longest_run and step.longest_context and L.has("ll_ragged_attention_mfma") and not os.environ.get("LL_RAGGED_ATTN_VALU")
            and L.lib().ll_ragged_attention_mfma_supported(dk, dv, L.dtype_code(dt)) and ks % 8 == 0 and vs % 8 == 0
            and k_cache.data_ptr() % 16 == 0 and v_cache.data_ptr() % 16 == 0):
        # 16-bit storage: the MFMA form -- tokens of a run as the columns of a wave (prompt portions, mixed steps), or, when every
        # sequence brings one decoded token, the query heads of a key/value head, with the context cut into partitions
        decode = step.longest_run == 1
        parts = -(-step.longest_context // int(L.lib().ll_ragged_attention_partition())) if decode else 1
        scratch = torch.empty(n * heads * parts * (2 + dv), dtype=torch.float32, device=q.device) if parts > 1 else None
        L.check(L.lib().ll_ragged_attention_mfma(
            q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), token_table.data_ptr(), token_table.stride(0),
            step.seq_req.data_ptr(), step.seq_start.data_ptr(), step.seq_first_pos.data_ptr(), L.ptr(sink), float(scale),
            out.data_ptr(), n, step.num_seqs, step.longest_run, step.longest_context, 1 if decode else 0, L.ptr(scratch), heads,
            kv_heads, dk, dv, ks, vs, int(window), int(keep_first), os_, L.dtype_code(dt), L.stream_ptr()), "ragged_attention_mfma")
        return out
    L.check(L.lib().ll_ragged_attention(q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), token_table.data_ptr(),
                                        token_table.stride(0), step.seq_req.data_ptr(), step.tok_seq.data_ptr(),
                                        step.tok_pos.data_ptr(), L.ptr(sink), float(scale), out.data_ptr(), n, heads, kv_heads, dk,
                                        dv, ks, vs, int(window), int(keep_first), os_, L.dtype_code(dt), L.stream_ptr()),
            "ragged_attention")
    return out


# ------------------------------------------------------------------------------------- #
# attention over a shared latent (csrc/latent_attn.hip): what surrounds the projections
# ------------------------------------------------------------------------------------- #
@torch.no_grad()
def latent_kv_prep(rows, kv_off: int, rank: int, rot: int, kv_norm_weight, eps: float, freq, pairs: int, amp: float, step, cache,
                   q_off: int = 0, q_rank: int = 0, q_norm_weight=None):
    """Rows of the fused input projection hold the key/value latent ``[rank]`` followed by the shared rotated key part
    ``[rot]`` at column ``kv_off``: the cache rows ``step.select`` of ``cache [rows, rank + rot]`` receive
    ``[RMS norm(latent) * weight | key part rotated at the token's position]``.  With ``q_rank`` the columns
    ``q_off .. q_off + q_rank`` (a query latent) are RMS-normed with ``q_norm_weight`` and returned ``[n, q_rank]``.
    ``freq`` fp32 ``[pairs]``: angle per position of pair i (entries 2i, 2i + 1); cos and sin are multiplied by ``amp``."""
    L.require_cuda(rows, cache, freq, kv_norm_weight)
    n, dt = rows.shape[0], rows.dtype
    if rows.dim() != 2 or rows.stride(1) != 1 or cache.dim() != 2 or cache.stride(1) != 1 or cache.dtype != dt \
            or cache.shape[1] != rank + rot:
        raise ValueError("latent_kv_prep: rows [n, ld] and cache [rows, rank + rot] in one dtype, unit inner strides")
    if freq.dtype != torch.float32 or freq.numel() < pairs or not freq.is_contiguous() or step.num_tokens != n:
        raise ValueError("latent_kv_prep: fp32 frequencies, one per rotated pair; a step of the rows' token count")
    for w, size in ((kv_norm_weight, rank), (q_norm_weight, q_rank)):
        if w is not None and (w.dtype != dt or w.numel() != size or not w.is_contiguous()):
            raise ValueError("latent_kv_prep: norm weights in the rows' dtype, one entry per normed column")
    q_out = torch.empty(n, q_rank, dtype=dt, device=rows.device) if q_rank else None
    L.check(L.lib().ll_latent_kv_prep(rows.data_ptr(), rows.stride(0), int(kv_off), int(rank), int(rot), kv_norm_weight.data_ptr(),
                                      float(eps), freq.data_ptr(), int(pairs), float(amp), step.tok_pos.data_ptr(),
                                      step.select.data_ptr(), cache.data_ptr(), cache.stride(0), int(q_off), int(q_rank),
                                      L.ptr(q_norm_weight), L.ptr(q_out), n, L.dtype_code(dt), L.stream_ptr()), "latent_kv_prep")
    return q_out


@torch.no_grad()
def rotate_pairs(q, q_off: int, rot: int, freq, pairs: int, amp: float, step, out, out_off: int):
    """``q [n, heads, w]`` (unit inner stride): the ``rot`` entries at ``q_off`` of every head, rotated pair by pair at the
    token's position, land at ``out[n, heads, w'][..., out_off : out_off + rot]`` (``out`` contiguous; it may be ``q`` itself
    with ``out_off == q_off``: every pair is read and written by one thread)."""
    L.require_cuda(q, out, freq)
    n, heads = q.shape[0], q.shape[1]
    if q.dim() != 3 or out.dim() != 3 or q.stride(2) != 1 or not out.is_contiguous() or out.shape[:2] != q.shape[:2] \
            or out.dtype != q.dtype or q_off + rot > q.shape[2] or out_off + rot > out.shape[2] or step.num_tokens != n:
        raise ValueError("rotate_pairs: q [n, heads, w] and a contiguous out [n, heads, w'] of one dtype")
    L.check(L.lib().ll_rotate_pairs(q.data_ptr(), q.stride(0), q.stride(1), int(q_off), int(rot), freq.data_ptr(), int(pairs),
                                    float(amp), step.tok_pos.data_ptr(), out.data_ptr(), out.shape[2], int(out_off), n, heads,
                                    L.dtype_code(q.dtype), L.stream_ptr()), "rotate_pairs")
    return out
