"""KV cache for the decode loop (plain ``KVCache`` of gbx_lm/models/cache.py:215-277; the rotating /
quantised / mamba caches and prompt-cache files are outside the hot path)."""
from __future__ import annotations

from typing import Any, List, Optional

import torch


def make_prompt_cache(model, max_kv_size: Optional[int] = None) -> List[Any]:
    """cache.py:11-36: defer to ``model.make_cache`` if present, else one KVCache per layer."""
    if hasattr(model, "make_cache"):
        return model.make_cache()
    if max_kv_size is not None:
        raise NotImplementedError("RotatingKVCache (max_kv_size) is outside the QuantizedLinear hot path")
    return [KVCache() for _ in range(len(model.layers))]


class KVCache:
    """Grows in ``step``-token blocks (cache.py:220-244); buffers are [B, n_kv, capacity, head_dim]."""

    def __init__(self, step: int = 256):
        self.keys = None
        self.values = None
        self.offset = 0
        self.step = step
        # graph-replayed decode (gbx_lm_amd/decode.py:GraphDecodeRunner): while ``static_active`` the write position is the
        # device-resident ``static_pos`` (int64 [1]) and attention runs over the whole buffer under a position mask, so one
        # captured launch sequence serves every step
        self.static_pos = None
        self.static_active = False

    @property
    def capacity(self) -> int:
        return 0 if self.keys is None else self.keys.shape[2]

    def reserve(self, n_new: int, like_k: torch.Tensor, like_v: torch.Tensor) -> None:
        """Make room for ``n_new`` more positions (same growth rule as update_and_fetch)."""
        prev = self.offset
        if self.keys is None or (prev + n_new) > self.keys.shape[2]:
            B, n_kv_heads, _, k_head_dim = like_k.shape
            v_head_dim = like_v.shape[3]
            n_steps = (self.step + n_new - 1) // self.step
            new_k = torch.zeros((B, n_kv_heads, n_steps * self.step, k_head_dim), dtype=like_k.dtype, device=like_k.device)
            new_v = torch.zeros((B, n_kv_heads, n_steps * self.step, v_head_dim), dtype=like_v.dtype, device=like_v.device)
            if self.keys is not None:
                if prev % self.step != 0:
                    self.keys = self.keys[..., :prev, :]
                    self.values = self.values[..., :prev, :]
                self.keys = torch.cat([self.keys, new_k], dim=2)
                self.values = torch.cat([self.values, new_v], dim=2)
            else:
                self.keys, self.values = new_k, new_v

    def update_and_fetch(self, keys: torch.Tensor, values: torch.Tensor):
        if self.static_active:                      # one new position at the device-resident index; shapes never change
            if (keys.is_cuda and keys.shape[2] == 1 and keys.dtype in (torch.bfloat16, torch.float16) and values.dtype == keys.dtype
                    and self.keys.is_contiguous() and self.values.is_contiguous()):
                from .. import ops                  # both caches in one launch (gbx_kv_append)
                ops.kv_append(self.keys, self.values, keys, values, self.static_pos)
            else:
                self.keys.index_copy_(2, self.static_pos, keys)
                self.values.index_copy_(2, self.static_pos, values)
            return self.keys, self.values
        prev = self.offset
        self.reserve(keys.shape[2], keys, values)
        self.offset += keys.shape[2]
        self.keys[..., prev:self.offset, :] = keys
        self.values[..., prev:self.offset, :] = values
        return self.keys[..., :self.offset, :], self.values[..., :self.offset, :]

    @property
    def state(self):
        if self.offset == self.keys.shape[2]:
            return self.keys, self.values
        return self.keys[..., :self.offset, :], self.values[..., :self.offset, :]

    @state.setter
    def state(self, v):
        self.keys, self.values = v
        self.offset = self.keys.shape[2]

    def is_trimmable(self):
        return True

    def trim(self, n):
        n = min(self.offset, n)
        self.offset -= n
        return n


class SequenceSlots:
    """Host-side table of the sequences a batched engine holds: ``length[s]`` is the number of tokens slot ``s`` has seen (the
    position of its next token), ``-1`` marks a free slot.  One table is shared by the per-layer caches of a model, so a position
    is advanced once per step, not once per layer.  Freed slots are handed out again lowest-first; the buffers behind a slot are
    not cleared -- a reader may only touch what the new owner's positions cover."""

    def __init__(self, n_slots: int = 1):
        self.length: List[int] = [-1] * n_slots
        self.listeners: List[Any] = []

    @property
    def n_slots(self) -> int:
        return len(self.length)

    def acquire(self) -> int:
        for s, n in enumerate(self.length):
            if n < 0:
                self.length[s] = 0
                return s
        self.length.append(0)
        for c in self.listeners:
            c.grow(len(self.length))
        return len(self.length) - 1

    def release(self, slot: int) -> None:
        if not (0 <= slot < len(self.length)) or self.length[slot] < 0:
            raise ValueError(f"slot {slot} is not held")
        self.length[slot] = -1

    def live_tokens(self) -> int:
        return sum(n for n in self.length if n > 0)


class WindowKVCache:
    """Keys / values of a sliding-window mixer for several sequences: one ring of ``window`` rows per slot, position ``p`` of a
    sequence lives in row ``p % window`` (a token that has left every later query's window is the one overwritten).  Buffers are
    token-major ``[slots, window, kv_heads * dim]`` so that a step's projection rows are appended as they are.  A step's own tokens
    are NOT read from the ring (a long portion would overwrite rows its earlier queries still need): the mixer reads them from
    the step's projection and appends after it has attended."""

    def __init__(self, window: int, slots: Optional[SequenceSlots] = None):
        self.window = int(window)
        self.slots = slots if slots is not None else SequenceSlots(1)
        self.slots.listeners.append(self)
        self.keys = None
        self.values = None

    @property
    def offset(self) -> int:                     # what generate_step reads: next position of the first sequence
        return max(self.slots.length[0], 0)

    def reserve(self, like_k: torch.Tensor, like_v: torch.Tensor) -> None:
        if self.keys is None:
            n = self.slots.n_slots
            self.keys = torch.zeros((n, self.window, like_k.shape[-1]), dtype=like_k.dtype, device=like_k.device)
            self.values = torch.zeros((n, self.window, like_v.shape[-1]), dtype=like_v.dtype, device=like_v.device)

    def grow(self, n_slots: int) -> None:
        if self.keys is not None and self.keys.shape[0] < n_slots:
            n = max(n_slots, 2 * self.keys.shape[0])
            for nm in ("keys", "values"):
                old = getattr(self, nm)
                new = torch.zeros((n,) + tuple(old.shape[1:]), dtype=old.dtype, device=old.device)
                new[:old.shape[0]] = old
                setattr(self, nm, new)

    def append_rows(self, k: torch.Tensor, v: torch.Tensor, slot: int, pos0: int) -> None:
        """Plain-torch append of one sequence's new rows (the HIP path appends a whole step in one launch)."""
        n, w = k.shape[0], self.window
        if n > w:
            k, v, pos0, n = k[n - w:], v[n - w:], pos0 + n - w, w
        rows = (torch.arange(pos0, pos0 + n, device=k.device) % w)
        self.keys[slot, rows] = k
        self.values[slot, rows] = v

    def is_trimmable(self):
        return False


class SlotKVCache:
    """Rows of a softmax-attention mixer for several sequences, token-major ``[slots, rows, width]``.  Position ``p`` of a sequence
    lives in row ``p`` while ``p < keep`` (the first tokens of a sequence, which a window mask may keep visible for ever) and in row
    ``keep + (p - keep) % ring`` afterwards.  Two shapes of the same table:

    * a window: ``ring = window`` rows are enough for every key a later query can still see;
    * no window (``window=None``): ``keep = 0`` and the ring is the whole capacity, which doubles when a sequence outgrows it
      (row = position while it fits, so a larger table is the old one copied in front).

    ``v_width = 0`` stores one row per token only (a mixer whose values are a part of its key rows: ``values`` is ``keys``).  As
    with ``WindowKVCache`` a step's own tokens are read from the step and appended after it has attended."""

    def __init__(self, k_width: int, v_width: int, window: Optional[int], keep: int = 0, slots: Optional[SequenceSlots] = None,
                 first_capacity: int = 256):
        self.k_width, self.v_width = int(k_width), int(v_width)
        self.window = None if window is None else int(window)
        self.keep = 0 if window is None else min(int(keep), 1 << 30)
        self.ring = first_capacity if window is None else self.window
        self.slots = slots if slots is not None else SequenceSlots(1)
        self.slots.listeners.append(self)
        self.keys = None
        self.values = None
        self.step_rows = None                     # the owner's key rows of the current step, for readers that share the table

    @property
    def offset(self) -> int:
        return max(self.slots.length[0], 0)

    @property
    def rows(self) -> int:
        return self.keep + self.ring

    def row_of(self, pos: torch.Tensor) -> torch.Tensor:
        return torch.where(pos < self.keep, pos, self.keep + (pos - self.keep) % self.ring)

    def _alloc(self, n_slots: int, dtype, device) -> None:
        self.keys = torch.zeros((n_slots, self.rows, self.k_width), dtype=dtype, device=device)
        self.values = torch.zeros((n_slots, self.rows, self.v_width), dtype=dtype, device=device) if self.v_width else self.keys

    def reserve(self, longest: int, dtype, device) -> None:
        """Room for sequences of up to ``longest`` tokens (allocates at first use; a windowed table never grows in rows)."""
        if self.window is None and longest > self.ring:
            old_k, old_v, old_rows = self.keys, self.values, self.ring
            while self.ring < longest:
                self.ring *= 2
            if old_k is not None:
                self._alloc(old_k.shape[0], old_k.dtype, old_k.device)
                self.keys[:, :old_rows] = old_k
                if self.v_width:
                    self.values[:, :old_rows] = old_v
        if self.keys is None:
            self._alloc(self.slots.n_slots, dtype, device)

    def ensure(self, longest: int) -> None:
        """Growth check for callers that replay captured launches (no allocation may happen inside a replay)."""
        if self.keys is not None:
            self.reserve(longest, self.keys.dtype, self.keys.device)

    def grow(self, n_slots: int) -> None:
        if self.keys is not None and self.keys.shape[0] < n_slots:
            old_k, old_v = self.keys, self.values
            self._alloc(max(n_slots, 2 * old_k.shape[0]), old_k.dtype, old_k.device)
            self.keys[:old_k.shape[0]] = old_k
            if self.v_width:
                self.values[:old_v.shape[0]] = old_v

    def stored(self, pos0: int) -> torch.Tensor:
        """Positions before ``pos0`` whose rows are still in the table, ascending."""
        first = max(self.keep, pos0 - self.ring)
        return torch.cat([torch.arange(0, min(self.keep, pos0)), torch.arange(first, max(first, pos0))])

    def append_rows(self, k: torch.Tensor, v: Optional[torch.Tensor], slot: int, pos0: int) -> None:
        """Plain-torch append of one sequence's new rows in order (the HIP path appends a whole step in one launch)."""
        n = k.shape[0]
        rows = self.row_of(torch.arange(pos0, pos0 + n))
        last = {int(r): i for i, r in enumerate(rows.tolist())}                  # a later row of the step takes the same place
        idx = torch.tensor(sorted(last.values()), dtype=torch.long)
        at = rows[idx].to(k.device)
        self.keys[slot, at] = k[idx.to(k.device)]
        if self.v_width:
            self.values[slot, at] = v[idx.to(k.device)]

    def is_trimmable(self):
        return False


class SharedLatentRows:
    """The cache entry of a mixer that attends over ANOTHER mixer's table (``source``, a ``SlotKVCache`` an earlier layer of the same
    step fills): it owns no buffer and appends nothing; positions before the step come from the source's table, the step's own rows
    from ``source.step_rows``."""

    def __init__(self, source: SlotKVCache):
        self.source = source
        self.slots = source.slots

    @property
    def keys(self):
        return self.source.keys

    @property
    def offset(self) -> int:
        return self.source.offset

    def ensure(self, longest: int) -> None:
        self.source.ensure(longest)

    def is_trimmable(self):
        return False


class SlotStateCache:
    """What a recurrent mixer carries from token to token, for several sequences: ``state`` fp32 ``[slots, heads, dv, dk]`` (one
    matrix per head; the key channels of one value channel lie side by side) and, for mixers with a short causal convolution in front, ``tail``
    ``[slots, taps - 1, channels]``: the last ``taps - 1`` inputs of the convolution in the activation dtype (oldest first).  A slot
    is not cleared when it is handed out again: a sequence whose step starts at position 0 starts from zeros (the kernels and the
    plain path test the position, never the buffer)."""

    def __init__(self, heads: int, dk: int, dv: int, channels: int = 0, taps: int = 0, slots: Optional[SequenceSlots] = None):
        self.heads, self.dk, self.dv = int(heads), int(dk), int(dv)
        self.channels, self.taps = int(channels), int(taps)
        self.slots = slots if slots is not None else SequenceSlots(1)
        self.slots.listeners.append(self)
        self.state = None
        self.tail = None

    @property
    def keys(self):                              # the buffer whose address a captured step depends on
        return self.state

    @property
    def offset(self) -> int:
        return max(self.slots.length[0], 0)

    def reserve(self, dtype, device) -> None:
        if self.state is None:
            n = self.slots.n_slots
            self.state = torch.zeros((n, self.heads, self.dv, self.dk), dtype=torch.float32, device=device)
            self.tail = torch.zeros((n, max(self.taps - 1, 0), self.channels), dtype=dtype, device=device)

    def grow(self, n_slots: int) -> None:
        if self.state is not None and self.state.shape[0] < n_slots:
            n = max(n_slots, 2 * self.state.shape[0])
            for nm in ("state", "tail"):
                old = getattr(self, nm)
                new = torch.zeros((n,) + tuple(old.shape[1:]), dtype=old.dtype, device=old.device)
                new[:old.shape[0]] = old
                setattr(self, nm, new)

    def is_trimmable(self):
        return False


class SlotRowCache:
    """One row of ``width`` values per slot: what a sequence's last token leaves for its next one (the previous token's id for a
    hashed pair embedding, the previous token's normed input for a token shift).  ``kind`` is "act" (the activation dtype of the
    first reserve), "f32" or "i64".  As with the other slot tables a slot is not cleared when it is handed out again: a sequence
    at position 0 has no previous token by position, never by the buffer's contents."""

    def __init__(self, width: int, kind: str = "act", slots: Optional[SequenceSlots] = None):
        if kind not in ("act", "f32", "i64"):
            raise ValueError("SlotRowCache: kind is act, f32 or i64")
        self.width, self.kind = int(width), kind
        self.slots = slots if slots is not None else SequenceSlots(1)
        self.slots.listeners.append(self)
        self.rows = None

    @property
    def keys(self):
        return self.rows

    @property
    def offset(self) -> int:
        return max(self.slots.length[0], 0)

    def reserve(self, dtype, device) -> None:
        if self.rows is None:
            dt = {"act": dtype, "f32": torch.float32, "i64": torch.int64}[self.kind]
            self.rows = torch.zeros((self.slots.n_slots, self.width), dtype=dt, device=device)

    def grow(self, n_slots: int) -> None:
        if self.rows is not None and self.rows.shape[0] < n_slots:
            new = torch.zeros((max(n_slots, 2 * self.rows.shape[0]), self.width), dtype=self.rows.dtype, device=self.rows.device)
            new[:self.rows.shape[0]] = self.rows
            self.rows = new

    def is_trimmable(self):
        return False


class CacheGroup:
    """The cache entry of a layer that carries more than one kind of state (say a token shift's row next to its mixer's table, or
    the two tables of two mixers side by side): named parts over ONE slot table.  ``buffers`` lists every device buffer a captured
    step depends on; ``ensure`` reaches the parts that can grow in rows."""

    def __init__(self, slots: SequenceSlots, **parts):
        self.slots = slots
        self.parts = dict(parts)
        for name, part in parts.items():
            if part is not None and part.slots is not slots:
                raise ValueError("CacheGroup: every part lives on the group's slot table")
            setattr(self, name, part)

    def _leaves(self):
        for part in self.parts.values():
            if isinstance(part, CacheGroup):
                yield from part._leaves()
            elif part is not None:
                yield part

    def buffers(self):
        out = []
        for c in self._leaves():
            for nm in ("keys", "values", "tail"):
                t = getattr(c, nm, None)
                if nm == "keys" or (t is not None and t.numel()):
                    out.append(t)
        return out

    @property
    def keys(self):                              # None until every part has its buffers
        bufs = self.buffers()
        return None if any(b is None for b in bufs) or not bufs else bufs[0]

    @property
    def offset(self) -> int:
        return max(self.slots.length[0], 0)

    def ensure(self, longest: int) -> None:
        for c in self._leaves():
            if hasattr(c, "ensure"):
                c.ensure(longest)

    def is_trimmable(self):
        return False
