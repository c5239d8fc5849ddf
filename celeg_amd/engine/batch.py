"""One step's batch: the rows, and the per-row and per-request numbers kernels need.

A step takes a list of entries, one per request: the request's next tokens (a
portion of its prompt, or one decoded token) and the places among them whose
logits are wanted.  The tokens of all entries are laid side by side into T rows.
The reference builds the same arrays for its packed passes, separately for a
prefill pass and a decode pass (src/backend/cuda/packed/batch_planner.cu:38-87);
here one batch holds both kinds.

All integer metadata travels to the device in ONE copy of one packed buffer.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch


TOKEN_FROM_DEVICE = -1        # a single-token entry whose token the device supplies


@dataclass
class StepEntry:
    slot: int                 # the request's slot in the cache manager
    start_pos: int            # position of tokens[0] in the request's sequence
    tokens: Sequence[int]     # [TOKEN_FROM_DEVICE]: the token the request sampled last, taken on the device
    want: Sequence[int] = ()  # indices into ``tokens`` whose logits are wanted


class StepBatch:
    """Device views (int32) into the packed buffer, plus host-side facts.

    token_ids[T], positions[T], token_seq[T] (which sequence a row belongs to),
    token_slot[T] (that entry's cache slot), cu_seqlens[S+1] (row offsets of the
    sequences), seq_slot[S], seq_start[S] (position of the sequence's first row),
    the sequences being the entries with those of a single token moved to the front,
    logit_rows[R] (rows whose logits are wanted), table_updates[g] ([1 + 3*cap]:
    a count, then (slot, logical page, physical page) triples) per cache group.
    """

    def __init__(self):
        self.n_tokens = 0
        self.n_seqs = 0
        self.n_logit_rows = 0
        self.n_real_seqs = 0
        self.max_seg_len = 0
        self.max_context_len = 0
        self.context_bound = 0    # set by whoever records the step for replay: the longest context the recording must serve
        self.decode_only = False
        self.single_rows = 0      # rows [0, single_rows) are entries of one token each
        self.entry_order: List[int] = []   # which entry each sequence of the layout is
        self.token_ids = self.positions = self.token_seq = self.token_slot = None
        self.cu_seqlens = self.seq_slot = self.seq_start = self.logit_rows = None
        self.table_updates: List[Optional[torch.Tensor]] = []
        self.table_update_caps: List[int] = []
        # host copies, for parts that plan on the host
        self.host: Dict[str, np.ndarray] = {}


def packed_layout(T: int, S: int, R: int, update_caps: Sequence[int]) -> Tuple[Dict[str, Tuple[int, int]], int]:
    """Offsets (in int32 elements) of every array in the packed buffer; each array
    starts at a multiple of 4 elements.  The layout depends only on the counts, so a
    captured graph of a fixed (T, S, R, caps) always finds its arrays in place."""
    fields = [("token_ids", T), ("positions", T), ("token_seq", T), ("token_slot", T),
              ("cu_seqlens", S + 1), ("seq_slot", S), ("seq_start", S), ("logit_rows", R)]
    for g, cap in enumerate(update_caps):
        fields.append((f"updates{g}", 1 + 3 * cap))
    layout = {}
    offset = 0
    for name, count in fields:
        layout[name] = (offset, count)
        offset += (count + 3) // 4 * 4
    return layout, offset


class BatchBuilder:
    """Packs entries on the host and ships them with one copy.  Two pinned staging
    buffers alternate, each guarded by an event, so a step's arrays are never
    overwritten while their copy is still in flight."""

    def __init__(self, device, capacity_ints: int, n_groups: int, pin: bool):
        self.device = torch.device(device)
        self.capacity = capacity_ints
        self.n_groups = n_groups
        self._stage = [torch.empty(capacity_ints, dtype=torch.int32, pin_memory=pin)
                       for _ in range(2)]
        self._events = [None, None]
        self._event_objects = [torch.cuda.Event(), torch.cuda.Event()] \
            if self.device.type == "cuda" else [None, None]
        self._iota = np.arange(max(capacity_ints, 1 << 16), dtype=np.int32)
        self._turn = 0
        self._layouts = {}      # (rows, requests, logit rows, update room) -> layout, size, device views
        self.device_buffer = torch.zeros(capacity_ints, dtype=torch.int32, device=self.device)

    def build(self, entries: Sequence[StepEntry], updates: Sequence[Sequence[Tuple[int, int, int]]],
              pad_to: Optional[int] = None, null_slot: int = 0,
              update_caps: Optional[Sequence[int]] = None,
              pad_singles_to: Optional[int] = None, last_rows_too: bool = False) -> StepBatch:
        """``pad_to``: for batches of single rows, the fixed number of rows of a captured
        graph; missing rows are filled with the null slot at position 0, and logits are
        produced for every row (wanted or not), so that the layout is the same every time.
        ``pad_singles_to``: for batches that hold portions (beside single rows or without),
        the fixed number of single rows of a captured graph; the missing ones are filled
        likewise, between the real single rows and the portions, and their logits come
        behind the wanted ones.  ``last_rows_too``: a portion that wants nothing gets the
        logits of its last row all the same, behind the wanted ones (a captured graph has a
        fixed number of logit rows)."""
        seg_lens = [len(e.tokens) for e in entries]
        S_real = len(entries)
        decode_only = all(n == 1 for n in seg_lens)
        if pad_to is not None and (not decode_only or pad_to < S_real):
            raise ValueError("only batches of single rows can be padded, and only upwards")
        n_single = sum(1 for n in seg_lens if n == 1)
        if pad_singles_to is not None and (decode_only or pad_to is not None or pad_singles_to < n_single):
            raise ValueError("pad_singles_to goes with batches that hold portions, and only upwards")
        n_pad = 0 if pad_singles_to is None else pad_singles_to - n_single
        T_real = S_real if decode_only else int(sum(seg_lens))
        S = (S_real if pad_to is None else pad_to) + n_pad
        T = (T_real if pad_to is None else pad_to) + n_pad
        # Rows are laid out with the entries of a single token first (their order kept), so
        # that kernels made for single rows can take them as one range also beside portions
        # of prompts; logits still come back in the order of the entries.
        order = list(range(S_real)) if decode_only else \
            sorted(range(S_real), key=lambda i: seg_lens[i] != 1)
        single_rows = S_real if decode_only else n_single
        if pad_to is not None:
            want_rows = list(range(T))
        else:
            first_row = [0] * S_real
            row = 0
            for i in order:
                if seg_lens[i] != 1 and row == n_single:
                    row += n_pad                 # the padding rows lie behind the real single rows
                first_row[i] = row
                row += seg_lens[i]
            want_rows = []
            for i, (e, n) in enumerate(zip(entries, seg_lens)):
                for w in e.want:
                    if not 0 <= int(w) < n:
                        raise ValueError(f"wanted place {w} is outside the entry's {n} tokens")
                    want_rows.append(first_row[i] + int(w))
            if last_rows_too:
                want_rows.extend(first_row[i] + n - 1 for i, (e, n) in enumerate(zip(entries, seg_lens))
                                 if n != 1 and not e.want)
            want_rows.extend(range(n_single, n_single + n_pad))
        R = len(want_rows)
        if update_caps is None:
            update_caps = [len(u) for u in updates]
        for u, cap in zip(updates, update_caps):
            if len(u) > cap:
                raise ValueError("more block-table updates than the step has room for")
        key = (T, S, R, tuple(update_caps))
        cached = self._layouts.get(key)
        if cached is None:
            if len(self._layouts) > 256:
                self._layouts.clear()
            cached = self._layouts[key] = packed_layout(T, S, R, update_caps) + ({},)
        layout, total, views = cached
        if total > self.capacity:
            raise ValueError(f"step metadata ({total} ints) exceeds the staging buffer "
                             f"({self.capacity} ints)")
        turn = self._turn
        self._turn ^= 1
        if self._events[turn] is not None:
            self._events[turn].synchronize()
        stage = self._stage[turn].numpy()

        def arr(name):
            off, count = layout[name]
            return stage[off:off + count]

        token_ids, positions = arr("token_ids"), arr("positions")
        token_seq, token_slot = arr("token_seq"), arr("token_slot")
        cu, seq_slot, seq_start = arr("cu_seqlens"), arr("seq_slot"), arr("seq_start")
        if decode_only:
            token_ids[:S_real] = [e.tokens[0] for e in entries]
            positions[:S_real] = [e.start_pos for e in entries]
            token_slot[:S_real] = [e.slot for e in entries]
            token_ids[S_real:] = 0
            positions[S_real:] = 0
            token_slot[S_real:] = null_slot
            token_seq[:] = self._iota[:T]
            cu[:] = self._iota[:S + 1]
            seq_slot[:] = token_slot
            seq_start[:] = positions
        else:
            row = 0
            cu[0] = 0
            seq = 0
            for e, n in ((entries[j], seg_lens[j]) for j in order):
                if n != 1 and n_pad and row == n_single:
                    token_ids[row:row + n_pad] = 0
                    positions[row:row + n_pad] = 0
                    token_seq[row:row + n_pad] = self._iota[seq:seq + n_pad]
                    token_slot[row:row + n_pad] = null_slot
                    seq_slot[seq:seq + n_pad] = null_slot
                    seq_start[seq:seq + n_pad] = 0
                    cu[seq + 1:seq + n_pad + 1] = self._iota[row + 1:row + n_pad + 1]
                    row += n_pad
                    seq += n_pad
                i = seq
                seq += 1
                token_ids[row:row + n] = e.tokens
                positions[row:row + n] = self._iota[e.start_pos:e.start_pos + n] \
                    if e.start_pos + n <= self._iota.size else np.arange(e.start_pos, e.start_pos + n)
                token_seq[row:row + n] = i
                token_slot[row:row + n] = e.slot
                seq_slot[i] = e.slot
                seq_start[i] = e.start_pos
                row += n
                cu[i + 1] = row
        arr("logit_rows")[:] = want_rows
        for g, u in enumerate(updates):
            a = arr(f"updates{g}")
            a[0] = len(u)
            if u:
                a[1:1 + 3 * len(u)] = np.asarray(u, dtype=np.int32).reshape(-1)
        self.device_buffer[:total].copy_(self._stage[turn][:total], non_blocking=True)
        if self.device.type == "cuda":
            ev = self._event_objects[turn]
            ev.record()
            self._events[turn] = ev

        b = StepBatch()
        b.n_tokens, b.n_seqs, b.n_logit_rows = T, S, R
        b.n_real_seqs = S_real
        b.max_seg_len = max(seg_lens) if seg_lens else 0
        b.max_context_len = max((e.start_pos + n for e, n in zip(entries, seg_lens)), default=0)
        b.decode_only = decode_only
        b.single_rows = S if decode_only else single_rows + n_pad
        b.entry_order = order

        def dev(name):       # the same views of the device buffer for the same layout
            view = views.get(name)
            if view is None:
                off, count = layout[name]
                view = views[name] = self.device_buffer[off:off + count]
            return view

        b.token_ids, b.positions = dev("token_ids"), dev("positions")
        b.token_seq, b.token_slot = dev("token_seq"), dev("token_slot")
        b.cu_seqlens, b.seq_slot, b.seq_start = dev("cu_seqlens"), dev("seq_slot"), dev("seq_start")
        b.logit_rows = dev("logit_rows")
        b.table_updates = [dev(f"updates{g}") for g in range(len(updates))]
        b.table_update_caps = list(update_caps)
        host_lens = [seg_lens[j] for j in order]
        host_lens = host_lens[:n_single] + [1] * n_pad + host_lens[n_single:] if n_pad \
            else host_lens + [1] * (S - S_real)
        b.host = {"seg_lens": np.asarray(host_lens, dtype=np.int32),
                  "seq_slot": seq_slot.copy(), "seq_start": seq_start.copy(),
                  "cu_seqlens": cu.copy(), "want_rows": np.asarray(want_rows, dtype=np.int32)}
        return b
