"""Ragged steps: the step function of models that take SEVERAL sequences per forward pass, each bringing a run of consecutive
tokens -- a portion of a prompt of any length, or the one token it decoded last -- against the cache and state that earlier
steps left.  Where :class:`SlotBatch` (slots.py) drives the padded-grid prefill / lockstep decode of the llama-shaped models,
this drives the layered models (model_layers.py): one flat token array, no padding, prompt portions next to decode tokens.

:class:`RaggedStep` is the metadata every kernel of such a step reads; :class:`RaggedRunner` owns the model, its
:class:`PagedStateCache` and the request slots, and is what both the generation engine (engine.py) and the trace replay
(trace_replay.py) call.
"""

from __future__ import annotations

from collections.abc import Sequence
from dataclasses import dataclass, field

import torch

from .paged_kv import PagedStateCache


@dataclass
class RaggedStep:
    """Device-side description of one step (all int32).  Per token: ``tok_seq`` (index of its sequence in the step), ``tok_pos``
    (position inside its sequence), ``select`` (cache row it writes).  Per sequence: ``seq_start [b + 1]`` (its run in the flat
    arrays), ``seq_first_pos`` (position of the run's first token), ``seq_slot`` / ``seq_req`` (its state slot = its row of the
    block and token tables), ``seq_parity`` (which half of a double-buffered state pair it reads)."""

    num_tokens: int
    num_seqs: int
    tok_seq: torch.Tensor
    tok_pos: torch.Tensor
    select: torch.Tensor
    seq_start: torch.Tensor
    seq_first_pos: torch.Tensor
    seq_slot: torch.Tensor
    seq_parity: torch.Tensor
    longest_run: int = 0       # most tokens a sequence brings (host copy; 0: not known)
    longest_context: int = 0   # longest sequence after this step (host copy; 0: not known)
    all_start: bool = False    # every sequence of the step starts at position 0 (host copy; False: not known)
    shared: dict = field(default_factory=dict, compare=False, repr=False)   # what layers of one forward pass compute once (rotation tables)

    @property
    def seq_req(self) -> torch.Tensor:
        return self.seq_slot


class _DecodeCell:
    """A captured decode step: the graph, the persistent packed step vectors it reads, the logits it leaves."""

    graph = None
    packed = None
    rows = None
    logits = None


class RaggedRunner:
    """Model + cache + request slots.  ``admit()`` hands out a slot, ``step()`` runs one ragged step and returns the logits of
    the asked rows, ``release()`` gives a request's blocks and slot back.  Nothing is kept per request on the host but its
    length and parity; blocks are popped and pushed on the device (``PagedStateCache``)."""

    def __init__(self, model, max_tokens: int, max_requests: int = 4, block_size: int = 64, device="cuda",
                 max_seq_len: int | None = None, capture_decode: bool = False):
        """``max_tokens``: the most tokens that live requests hold at any time, each request's count rounded up to a multiple
        of ``block_size``: the block pool is made for that many (plus the junk block), not for ``max_requests`` full-length
        sequences."""
        self.model = model
        self.device = torch.device(device)
        self.block_size = block_size
        blocks = -(-max_tokens // block_size)
        self.max_seq_len = (max_seq_len if max_seq_len is not None else blocks * block_size)
        self.max_seq_len = -(-self.max_seq_len // block_size) * block_size
        self.max_requests = max_requests
        self.cache = PagedStateCache(model.cache_runs(), blocks + 1, block_size, self.device, max_requests, self.max_seq_len,
                                     model.dtype, previous_token=bool(getattr(model, "needs_previous_token", False)))
        self.vocab_size = int(getattr(getattr(model, "geo", None), "vocab_size", 0))
        self.token_table = torch.zeros(max_requests, self.max_seq_len, dtype=torch.int32, device=self.device)
        self.total_blocks = blocks
        self._free_slots = list(range(max_requests))
        self._len: dict[int, int] = {}
        self._parity: dict[int, int] = {}
        self._all_start = False    # the step planned last: every sequence at position 0
        # captured decode steps (opt-in): one hipGraph per (slots riding, context partitions) cell, see _decode_cell
        self.capture_decode = bool(capture_decode)
        self._cells: dict[tuple, "_DecodeCell"] = {}
        self._sightings: dict[tuple, int] = {}
        self.replays = 0

    # ------------------------------------------------------------------ requests ---- #
    @property
    def free_slots(self) -> int:
        return len(self._free_slots)

    def blocks_held(self) -> int:
        return sum(-(-n // self.block_size) for n in self._len.values())

    def blocks_for(self, tokens: int) -> int:
        return -(-tokens // self.block_size)

    def length(self, slot: int) -> int:
        return self._len[slot]

    def admit(self) -> int:
        if not self._free_slots:
            raise RuntimeError(f"all {self.max_requests} request slots are taken")
        slot = self._free_slots.pop(0)
        self._len[slot] = 0
        self._parity[slot] = 0
        return slot

    def release(self, slots: Sequence[int]) -> None:
        slots = [s for s in slots if s in self._len]
        if not slots:
            return
        self.cache.release(torch.tensor(slots, dtype=torch.int32, device=self.device))
        for s in slots:
            del self._len[s], self._parity[s]
            self._free_slots.append(s)

    # ------------------------------------------------------------------ one step ---- #
    def _plan(self, entries: Sequence[tuple[int, Sequence[int]]]):
        """``entries``: ``(slot, next tokens)`` per sequence, every slot at most once.  Checks the step against the pool, builds
        its vectors as host lists and advances the host-side lengths and parities."""
        if not entries:
            raise ValueError("an empty step")
        slots = [s for s, _ in entries]
        if len(set(slots)) != len(slots):
            raise ValueError("a request rides at most once in a step")
        counts = [len(t) for _, t in entries]
        if min(counts) < 1:
            raise ValueError("every entry brings at least one token")
        if self.vocab_size and not all(0 <= int(t) < self.vocab_size for _, toks in entries for t in toks):
            raise ValueError(f"token ids lie in 0 .. {self.vocab_size - 1}")
        first = [self._len[s] for s in slots]
        new_len = [f + c for f, c in zip(first, counts)]
        if max(new_len) > self.max_seq_len:
            raise RuntimeError(f"a sequence of {max(new_len)} tokens exceeds the cache's {self.max_seq_len}")
        need = sum(self.blocks_for(n) - self.blocks_for(f) for n, f in zip(new_len, first))
        if self.blocks_held() + need > self.total_blocks:
            raise RuntimeError(f"the block pool is exhausted: {self.blocks_held()} of {self.total_blocks} blocks held, {need} more asked")
        starts, tok_seq, tok_pos, pick, tokens = [0], [], [], [], []
        longest = max(counts)
        for i, ((_, toks), f, c) in enumerate(zip(entries, first, counts)):
            starts.append(starts[-1] + c)
            tok_seq += [i] * c
            tok_pos += range(f, f + c)
            pick += range(i * longest + longest - c, (i + 1) * longest)
            tokens += [int(t) for t in toks]
        parts = [tok_seq, tok_pos, starts, first, slots, [self._parity[s] for s in slots], new_len, pick, tokens]
        for s, n in zip(slots, new_len):
            self._len[s] = n
            self._parity[s] ^= 1
        self._all_start = not any(first)
        return parts, longest, max(new_len)

    @staticmethod
    def _views(packed: torch.Tensor, sizes):
        views, at = [], 0
        for n in sizes:
            views.append(packed[at:at + n])
            at += n
        return views

    def build_step(self, entries: Sequence[tuple[int, Sequence[int]]]) -> tuple[RaggedStep, torch.Tensor]:
        """The step's device vectors: every one of them crosses to the device in ONE copy (a packed int32 tensor, sliced into
        views); blocks for the new tokens are reserved on the device."""
        parts, longest, longest_context = self._plan(entries)
        packed = torch.tensor([v for part in parts for v in part], dtype=torch.int32).to(self.device, non_blocking=True)
        return self._step_from(packed, [len(p) for p in parts], len(entries), longest, longest_context)

    def _step_from(self, packed, sizes, num_seqs, longest, longest_context):
        v_tok_seq, v_tok_pos, v_starts, v_first, v_slots, v_parity, v_new_len, v_pick, v_tokens = self._views(packed, sizes)
        rows = self.cache.extend(v_slots, v_new_len, longest, self.token_table)
        select = rows.reshape(-1)[v_pick].contiguous() if longest > 1 else rows.reshape(-1)
        step = RaggedStep(num_tokens=v_tokens.numel(), num_seqs=num_seqs, tok_seq=v_tok_seq, tok_pos=v_tok_pos, select=select,
                          seq_start=v_starts, seq_first_pos=v_first, seq_slot=v_slots, seq_parity=v_parity, longest_run=longest,
                          longest_context=longest_context, all_start=self._all_start and longest > 1)
        return step, v_tokens

    @torch.no_grad()
    def step(self, entries: Sequence[tuple[int, Sequence[int]]], logits_rows: Sequence[int] | None = None, *,
             collect_layers: list | None = None) -> torch.Tensor | None:
        """Run the entries as ONE batch.  ``logits_rows``: flat token indices (in entry order) whose logits are wanted; ``None``
        = the last token of every entry; an empty list = none (the step still fills cache and state).  Returns
        ``[rows, vocab]`` logits in the model's dtype, or ``None``."""
        if logits_rows is None:
            logits_rows, at = [], 0
            for _, toks in entries:
                at += len(toks)
                logits_rows.append(at - 1)
        logits_rows = list(logits_rows)
        if (self.capture_decode and collect_layers is None and all(len(t) == 1 for _, t in entries)
                and logits_rows == list(range(len(entries)))):
            return self._decode_step_captured(entries)
        step, token_ids = self.build_step(entries)
        rows = torch.tensor(logits_rows, dtype=torch.long, device=self.device) if logits_rows else None
        return self.model(token_ids, step, self.cache, self.token_table, logits_rows=rows, collect_layers=collect_layers)

    # ------------------------------------------------------------------ captured decode steps ---- #
    def _decode_step_captured(self, entries):
        """A step in which every sequence brings its one decoded token and every row's logits are wanted.  Such steps repeat
        with the same slots for as long as nobody finishes: the SECOND time a (slots, context partitions) cell is seen its
        launch list is captured as one hipGraph over persistent step vectors, and from then on a step is one small host-to-
        device copy plus one graph launch.  The first sighting runs eagerly (which also sizes every workspace the capture
        needs).  The returned logits live in the graph's memory: use them before the next step of the same cell."""
        from .. import _lib as L

        part = int(L.lib().ll_ragged_attention_partition()) if L.has("ll_ragged_attention_partition") else 256
        parts, longest, longest_context = self._plan(entries)
        key = (tuple(s for s, _ in entries), -(-longest_context // part))
        host = torch.tensor([v for p in parts for v in p], dtype=torch.int32)
        cell = self._cells.get(key)
        if cell is None:
            self._sightings[key] = self._sightings.get(key, 0) + 1
            if self._sightings[key] < 2:
                step, token_ids = self._step_from(host.to(self.device), [len(p) for p in parts], len(entries), 1, longest_context)
                rows = torch.arange(len(entries), device=self.device)
                return self.model(token_ids, step, self.cache, self.token_table, logits_rows=rows)
            cell = self._capture_cell(key, host, [len(p) for p in parts], len(entries), key[1] * part)
        cell.packed.copy_(host)   # (pageable source: the copy has left the host buffer when this returns)
        cell.graph.replay()
        self.replays += 1
        return cell.logits

    def _capture_cell(self, key, host, sizes, num_seqs, context_bound):
        while len(self._cells) >= 8:                      # a handful of cells at a time: the oldest goes
            self._cells.pop(next(iter(self._cells)))
        cell = _DecodeCell()
        cell.packed = host.to(self.device)
        cell.rows = torch.arange(num_seqs, device=self.device)
        torch.cuda.synchronize()
        cell.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(cell.graph):
            step, token_ids = self._step_from(cell.packed, sizes, num_seqs, 1, context_bound)
            cell.logits = self.model(token_ids, step, self.cache, self.token_table, logits_rows=cell.rows)
        self._cells[key] = cell
        self._sightings.pop(key, None)
        return cell

    def check_errors(self) -> None:
        """Synchronising read of the block pool's sticky error word."""
        err = self.cache.error
        if err:
            raise RuntimeError(f"paged cache reported error bits {err:#x} (1: too few free blocks, 2: a request outgrew its table row)")
