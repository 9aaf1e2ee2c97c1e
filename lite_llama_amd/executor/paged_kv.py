"""Block-granular KV pool on the device (extension -- the reference's pool is token-granular with the
paging TODO at executor/kv_cache_manager.py:211).  Same storage as :class:`KVPool` (one ``[rows, 2*Hkv, D]`` tensor per
layer, rows = blocks x block_size), handed out in blocks; the per-token table the kernels read
(``b_req_tokens_table``) is derived on the device by ``ll_kv_paged_extend``, so the attention / KV-write kernels and
their results are those of token attention.  Nothing is read back: admission, the per-step append and release are
stream-ordered launches (the append sits inside the captured decode step); the host looks at ``free_blocks`` /
``error`` only when it chooses to synchronise."""

from __future__ import annotations

import torch

from .. import _lib as L


class PagedKVPool:
    def __init__(self, num_layers: int, num_blocks: int, block_size: int, num_kv_heads: int, head_dim: int, device,
                 max_requests: int, max_seq_len: int, dtype=torch.float16):
        if block_size < 1 or num_blocks < 2:
            raise ValueError("PagedKVPool needs block_size >= 1 and num_blocks >= 2 (one block is the junk block)")
        self.block_size, self.num_blocks, self.device = block_size, num_blocks, device
        self.max_requests, self.max_seq_len = max_requests, max_seq_len
        self.max_tokens = num_blocks * block_size
        self.kv_buffer = self._make_buffers(num_layers, num_kv_heads, head_dim, dtype)
        self.blocks_per_request = (max_seq_len + block_size - 1) // block_size
        self.free_stack = torch.empty(num_blocks - 1, dtype=torch.int32, device=device)
        self.state = torch.zeros(2, dtype=torch.int32, device=device)          # [free blocks, error flags]
        self.block_table = torch.zeros(max_requests, self.blocks_per_request, dtype=torch.int32, device=device)
        self.req_blocks = torch.zeros(max_requests, dtype=torch.int32, device=device)
        self.reset()

    def _make_buffers(self, num_layers, num_kv_heads, head_dim, dtype):
        return [torch.zeros(self.max_tokens, 2 * num_kv_heads, head_dim, dtype=dtype, device=self.device)
                for _ in range(num_layers)]

    def reset(self) -> None:
        L.check(L.lib().ll_kv_paged_reset(self.free_stack.data_ptr(), self.state.data_ptr(), self.req_blocks.data_ptr(),
                                          self.num_blocks, self.max_requests, L.stream_ptr()), "kv_paged_reset")

    def _extend(self, req_idx, lens, len_bias, grid_len, from_end, token_table, out=None):
        n = req_idx.numel()
        L.require_cuda(req_idx, lens, token_table)
        if req_idx.dtype != torch.int32 or lens.dtype != torch.int32 or token_table.dtype != torch.int32:
            raise ValueError("PagedKVPool: request indices, lengths and the token table must be int32")
        if token_table.stride(1) != 1 or not req_idx.is_contiguous() or not lens.is_contiguous():
            raise ValueError("PagedKVPool: the token table must be row-major, indices and lengths contiguous")
        select = out if out is not None else torch.empty(n * grid_len, dtype=torch.int32, device=self.device)
        if select.dtype != torch.int32 or select.numel() != n * grid_len or not select.is_contiguous():
            raise ValueError("PagedKVPool: the row output must be a contiguous int32 tensor of n * grid_len entries")
        L.check(L.lib().ll_kv_paged_extend(
            self.free_stack.data_ptr(), self.state.data_ptr(), self.block_table.data_ptr(), self.block_table.stride(0),
            self.req_blocks.data_ptr(), req_idx.data_ptr(), lens.data_ptr(), len_bias, n, self.block_size, grid_len,
            from_end, token_table.data_ptr(), token_table.stride(0), select.data_ptr(), self.num_blocks, L.stream_ptr()),
            "kv_paged_extend")
        return select

    @torch.no_grad()
    def admit(self, req_idx: torch.Tensor, lens: torch.Tensor, grid_len: int, token_table: torch.Tensor) -> torch.Tensor:
        """Blocks for ``lens[i]`` tokens of every listed request + the rows of the padded prefill grid ``[n, grid_len]``
        (``cur_select_index``; pad positions name junk rows); fills ``token_table[req, :len]``."""
        return self._extend(req_idx, lens, 0, grid_len, 0, token_table)

    @torch.no_grad()
    def append(self, req_idx: torch.Tensor, seq_len: torch.Tensor, token_table: torch.Tensor, out=None) -> torch.Tensor:
        """The decode step's row: position ``seq_len[i] - 1`` of every listed request (a new block is popped when the
        position opens one); writes ``token_table[req, seq_len - 1]`` and returns / fills ``cur_select_index``."""
        return self._extend(req_idx, seq_len, 0, 1, 1, token_table, out=out)

    @torch.no_grad()
    def release(self, req_idx: torch.Tensor) -> None:
        L.require_cuda(req_idx)
        L.check(L.lib().ll_kv_paged_release(self.free_stack.data_ptr(), self.state.data_ptr(), self.block_table.data_ptr(),
                                            self.block_table.stride(0), self.req_blocks.data_ptr(), req_idx.data_ptr(),
                                            req_idx.numel(), L.stream_ptr()), "kv_paged_release")

    # host-visible (synchronising) views
    @property
    def free_blocks(self) -> int:
        return int(self.state[0].item())

    @property
    def error(self) -> int:
        """0, or flags: 1 = a call found too few free blocks (it allocated nothing), 2 = a request outgrew max_seq_len."""
        return int(self.state[1].item())

    def snapshot(self):
        return self.state.clone(), self.req_blocks.clone(), self.block_table.clone()

    def restore(self, snap) -> None:
        """Undo appends made since ``snapshot`` (pops only move the stack top: the stack itself is intact)."""
        self.state.copy_(snap[0])
        self.req_blocks.copy_(snap[1])
        self.block_table.copy_(snap[2])


class PagedStateCache(PagedKVPool):
    """Cache of a model whose layer RUNS differ in what they keep per sequence (a layer that runs several times in a forward
    pass keeps one set per run): attention runs own ``(K [rows, kv_heads, dk], V [rows, kv_heads, dv])`` in the block pool --
    key and value widths may differ --, latent-attention runs one row ``[latent | rotated key part]`` per token, recurrent runs own a fixed-size fp32 state ``[slots, heads, dk, dv]``, and any run may
    own a token-shift row pair ``[2, slots, width]`` (double-buffered by the sequence's parity).  An attention run with a short
    convolution in front of it carries the projected rows of a sequence's last positions, ``[2, slots, taps - 1, channels]``,
    double-buffered the same way; a run whose values are blended with those of an earlier run names that run in
    ``value_source``; a model whose input depends on the previous token keeps it per sequence in ``prev_token [2, slots]``.  One block allocator, one
    block table and one per-token row table serve all attention runs; a sequence's slot is its row of those tables, so blocks
    and slots are handed out and given back together.  Fixed-size state is never cleared: the kernels start a sequence whose
    run begins at position 0 from zeros, whatever an earlier owner of the slot left."""

    def __init__(self, runs, num_blocks: int, block_size: int, device, max_requests: int, max_seq_len: int, dtype,
                 previous_token: bool = False):
        """``runs``: one mapping per layer run: ``{"kind": "attention", "kv_heads", "dk", "dv"}``, ``{"kind": "latent", "rank",
        "rot"}`` or ``{"kind": "recurrent", "heads", "dk", "dv"}``, each with an optional ``"shift_width"``; attention runs may
        add ``"conv_taps"`` / ``"conv_channels"`` (rows carried for a convolution of that many taps), ``"value_mix": True``
        (the first such run is the value source of the later ones) and ``"state": (heads, dk, dv)`` (a recurrence that runs
        beside the attention keeps its fp32 state in the same run).  ``previous_token``: keep each sequence's last token."""
        self.runs = [dict(r) for r in runs]
        self.dtype = dtype
        self.prev_token = torch.zeros(2, max_requests, dtype=torch.int32, device=device) if previous_token else None
        super().__init__(len(self.runs), num_blocks, block_size, 1, 1, device, max_requests, max_seq_len, dtype)

    def _make_buffers(self, num_layers, num_kv_heads, head_dim, dtype):
        dev, slots = self.device, self.max_requests
        self.recurrent, self.shift, self.conv, self.value_source = [], [], [], []
        buffers = []
        first_mix = None
        for index, r in enumerate(self.runs):
            taps = int(r.get("conv_taps", 0)) if r["kind"] == "attention" else 0
            self.conv.append(torch.zeros(2, slots, taps - 1, int(r["conv_channels"]), dtype=dtype, device=dev) if taps > 1 else None)
            mixes = r["kind"] == "attention" and bool(r.get("value_mix"))
            self.value_source.append(first_mix if mixes else None)
            if mixes and first_mix is None:
                first_mix = index
            elif mixes and (self.runs[first_mix]["kv_heads"], self.runs[first_mix]["dv"]) != (r["kv_heads"], r["dv"]):
                raise ValueError(f"layer run {index} blends its values with those of run {first_mix}, whose shape differs")
            if r["kind"] == "attention":
                buffers.append((torch.zeros(self.max_tokens, r["kv_heads"], r["dk"], dtype=dtype, device=dev),
                                torch.zeros(self.max_tokens, r["kv_heads"], r["dv"], dtype=dtype, device=dev)))
                # a mixer that runs a recurrence beside its attention keeps both: "state": (heads, dk, dv)
                self.recurrent.append(torch.zeros(slots, *r["state"], dtype=torch.float32, device=dev) if r.get("state") else None)
            elif r["kind"] == "latent":
                # one row [latent (rank) | rotated key part (rot)] per token: the keys of ONE key/value head; the values are the
                # latent columns of the same rows (a row-strided view, nothing is stored twice)
                rows = torch.zeros(self.max_tokens, 1, r["rank"] + r["rot"], dtype=dtype, device=dev)
                buffers.append((rows, rows[:, :, :r["rank"]]))
                self.recurrent.append(None)
            elif r["kind"] == "recurrent":
                buffers.append(None)
                self.recurrent.append(torch.zeros(slots, r["heads"], r["dk"], r["dv"], dtype=torch.float32, device=dev))
            else:
                raise ValueError(f"unknown layer-run kind {r['kind']!r}")
            w = int(r.get("shift_width", 0))
            self.shift.append(torch.zeros(2, slots, w, dtype=torch.float32, device=dev) if w else None)
        return buffers

    def extend(self, req_idx: torch.Tensor, new_lens: torch.Tensor, longest_run: int, token_table: torch.Tensor) -> torch.Tensor:
        """Blocks for every listed request up to ``new_lens[i]`` tokens; returns the cache rows of each request's LAST
        ``longest_run`` positions ``[n, longest_run]`` (a request that brings fewer tokens uses the tail of its row)."""
        return self._extend(req_idx, new_lens, 0, longest_run, 1, token_table).view(req_idx.numel(), longest_run)

    def state_bytes(self) -> int:
        total, seen = 0, set()
        for group in (self.kv_buffer, self.recurrent, self.shift, self.conv, [self.prev_token]):
            for t in group:
                for u in (t if isinstance(t, tuple) else (t,)):
                    if u is not None and u.untyped_storage().data_ptr() not in seen:   # (a view of counted rows adds nothing)
                        seen.add(u.untyped_storage().data_ptr())
                        total += u.untyped_storage().nbytes()
        return total
