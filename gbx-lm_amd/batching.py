"""Ragged step batches and the slot scheduler of models that hold per-sequence state in slots (models/cache.py:SequenceSlots).

A step is a list of (sequence, its next tokens): sequences that start and sequences that go on by one token mix freely, each
with its own position.  The tokens of a step are laid out back to back -- no padding rows exist, so nothing a sequence computes
depends on the lengths of its neighbours -- and every kernel finds a token's sequence, slot and position through the small
descriptor tables built here once per step (one host-to-device copy).

``BatchScheduler`` is the engine above it: it owns the caches, hands slots out and takes them back, runs a step through
``model.forward_tokens`` and the output head on the rows that are asked for, and generates for several prompts at once
(``generate``) with the same sampler interface as ``generate_step``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Dict, Iterable, List, Optional, Sequence, Tuple

import torch

from . import env


@dataclass
class StepBatch:
    """One step's layout.  Host lists (one item per sequence of the step) and their device images."""
    slot: List[int]
    pos0: List[int]                 # position of the sequence's first new token
    n_new: List[int]
    total: int                      # tokens of the step
    seq: torch.Tensor               # int32 [B, 4]: slot, pos0, n_new, first row of the sequence in the step
    tok: torch.Tensor               # int32 [T, 2]: sequence of the step a row belongs to, its position
    q_tile: int = 0                 # query rows per tile of ``tiles``
    tiles: Optional[torch.Tensor] = None   # int32 [n_tiles, 2]: sequence of the step, first row of the tile inside it

    @property
    def decode_only(self) -> bool:
        return all(n == 1 for n in self.n_new)

    @staticmethod
    def build(slot: Sequence[int], pos0: Sequence[int], n_new: Sequence[int], device, q_tile: int = 128) -> "StepBatch":
        rows, seq, tok, tiles = 0, [], [], []
        for b, (s, p, n) in enumerate(zip(slot, pos0, n_new)):
            if n <= 0:
                raise ValueError("a sequence of a step brings at least one token")
            seq.append((s, p, n, rows))
            tok.extend((b, p + i) for i in range(n))
            tiles.extend((b, t) for t in range(0, n, q_tile))
            rows += n
        packed = torch.tensor([v for r in seq for v in r] + [v for r in tok for v in r] + [v for r in tiles for v in r],
                              dtype=torch.int32)
        if torch.device(device).type == "cuda":
            packed = packed.pin_memory().to(device, non_blocking=True)
        nb, nt = len(seq), len(tok)
        return StepBatch(list(slot), list(pos0), list(n_new), rows, packed[:4 * nb].view(nb, 4),
                         packed[4 * nb:4 * nb + 2 * nt].view(nt, 2), q_tile, packed[4 * nb + 2 * nt:].view(-1, 2))


class _DecodeGraph:
    """One decode step (every sequence brings one token) of a fixed set of slots, captured in a HIP graph.  Tokens and the step's
    descriptor tables live in one static device buffer that a single host-to-device copy refreshes before each replay; the
    launches, their grids and every pointer they read are the same from step to step, only positions and tokens change."""

    def __init__(self, sched: "BatchScheduler", slots: Tuple[int, ...]):
        self.slots = slots
        b = len(slots)
        dev = sched.device
        # int64 words: tokens [b] | seq [b, 4] as int32 pairs | tok [b, 2] | tiles [b, 2]
        self.words = b + 2 * b + b + b
        self.static = torch.zeros((self.words,), dtype=torch.int64, device=dev)
        self.pinned = [torch.zeros((self.words,), dtype=torch.int64, pin_memory=True) for _ in range(2)]
        self.copied = [None, None]
        self.turn = 0
        i32 = self.static.view(torch.int32)
        self.tokens = self.static[:b]
        self.batch = StepBatch(list(slots), [0] * b, [1] * b, b, i32[2 * b:6 * b].view(b, 4), i32[6 * b:8 * b].view(b, 2), 128,
                               i32[8 * b:10 * b].view(b, 2))
        self.graph = None
        self.logits = None

    def fill(self, tokens: Sequence[int], pos0: Sequence[int]) -> None:
        k = self.turn % 2
        self.turn += 1
        if self.copied[k] is not None:
            self.copied[k].synchronize()                 # the copy that last read this host buffer has run
        host = self.pinned[k]
        b = len(self.slots)
        host[:b] = torch.tensor(tokens, dtype=torch.int64)
        i32 = host.view(torch.int32)
        i32[2 * b:6 * b] = torch.tensor([v for i, (s, p) in enumerate(zip(self.slots, pos0)) for v in (s, p, 1, i)], dtype=torch.int32)
        i32[6 * b:8 * b] = torch.tensor([v for i, p in enumerate(pos0) for v in (i, p)], dtype=torch.int32)
        i32[8 * b:10 * b] = torch.tensor([v for i in range(b) for v in (i, 0)], dtype=torch.int32)
        self.static.copy_(host, non_blocking=True)
        self.copied[k] = torch.cuda.Event()
        self.copied[k].record(torch.cuda.current_stream(self.static.device))
        self.batch.pos0 = list(pos0)

    def run(self, sched: "BatchScheduler") -> torch.Tensor:
        if self.graph is None:
            torch.cuda.synchronize(sched.device)
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                self.logits = sched.model.logits(sched.model.forward_tokens(self.tokens, self.batch, sched.caches))
            self.graph = g
        self.graph.replay()
        return self.logits


class BatchScheduler:
    """Sequences in slots, stepped together.  ``step`` takes what each live sequence brings next and returns the logits of the rows
    that are asked for; ``release`` gives a finished sequence's slot back.  ``max_tokens`` bounds the tokens live sequences may hold
    (a request past it is refused before anything is written)."""

    def __init__(self, model, max_tokens: Optional[int] = None):
        self.model = model
        self.caches = model.make_cache()
        self.slots = self.caches[0].slots
        self.slots.length[0] = -1                       # make_cache hands out slot 0 for the one-sequence loop; nothing holds it here
        self.max_tokens = max_tokens
        self.slot_of: Dict[object, int] = {}
        self.device = next(model.parameters()).device
        # decode-only steps of a set of slots that keeps coming back are replayed from a HIP graph (captured at its third step)
        self.use_graphs = self.device.type == "cuda" and env.flag("GBX_STEP_GRAPH")
        self._graphs: Dict[Tuple[int, ...], _DecodeGraph] = {}
        self._seen: Dict[Tuple[int, ...], int] = {}
        self._buffers = None

    def position(self, seq_id) -> int:
        return self.slots.length[self.slot_of[seq_id]]

    def release(self, seq_id) -> None:
        self.slots.release(self.slot_of.pop(seq_id))

    @torch.no_grad()
    def step(self, entries: Sequence[Tuple[object, Sequence[int]]], want: Optional[Sequence[Sequence[int]]] = None) -> torch.Tensor:
        """``entries``: (sequence id, next tokens); an id not seen before starts a sequence at position 0.  ``want[i]``: places among
        entry i's tokens whose logits are returned (default: the last one), in the order of entries and places.  Returns fp32
        [wanted, vocab]."""
        if not entries:
            return torch.empty((0, 0))
        new_tokens = sum(len(t) for _, t in entries)
        if self.max_tokens is not None and self.slots.live_tokens() + new_tokens > self.max_tokens:
            raise RuntimeError(f"step would hold {self.slots.live_tokens() + new_tokens} tokens, more than max_tokens={self.max_tokens}")
        if len({i for i, _ in entries}) != len(entries):
            raise ValueError("a sequence appears twice in one step")
        for seq_id, _ in entries:
            if seq_id not in self.slot_of:
                self.slot_of[seq_id] = self.slots.acquire()
        slot = [self.slot_of[i] for i, _ in entries]
        pos0 = [self.slots.length[s] for s in slot]
        n_new = [len(t) for _, t in entries]
        if self.use_graphs and all(n == 1 for n in n_new) and len(slot) <= 256:
            logits = self._graph_step(tuple(slot), [ts[0] for _, ts in entries], pos0)
            if logits is not None:
                for s in slot:
                    self.slots.length[s] += 1
                rows = [i for i in range(len(slot)) if want is None or len(want[i])]
                if any(p != 0 for i in rows if want is not None for p in want[i]):
                    raise ValueError("a wanted place lies outside the entry's tokens")
                if not rows:
                    return torch.empty((0, self.model.args.vocab), dtype=torch.float32, device=self.device)
                return logits.index_select(0, torch.tensor(rows, dtype=torch.long, device=self.device)).float()
        batch = StepBatch.build(slot, pos0, n_new, self.device)
        tokens = torch.tensor([t for _, ts in entries for t in ts], dtype=torch.long)
        if self.device.type == "cuda":
            tokens = tokens.pin_memory().to(self.device, non_blocking=True)
        hidden = self.model.forward_tokens(tokens, batch, self.caches)
        for s, n in zip(slot, n_new):
            self.slots.length[s] += n
        rows, first = [], 0
        for i, n in enumerate(n_new):
            places = [n - 1] if want is None else want[i]
            for p in places:
                if not 0 <= p < n:
                    raise ValueError("a wanted place lies outside the entry's tokens")
                rows.append(first + p)
            first += n
        if not rows:
            return torch.empty((0, self.model.args.vocab), dtype=torch.float32, device=self.device)
        idx = torch.tensor(rows, dtype=torch.long, device=self.device)
        return self.model.logits(hidden.index_select(0, idx)).float()

    def _graph_step(self, slots: Tuple[int, ...], tokens: Sequence[int], pos0: Sequence[int]) -> Optional[torch.Tensor]:
        """Replay (or, at the third step of this set of slots, capture) the decode graph; None: run the step eagerly."""
        longest = max(pos0) + 1
        for c in self.caches:                            # tables without a window grow on the host, never inside a replay
            if hasattr(c, "ensure"):
                c.ensure(longest)
        buffers = tuple(b.data_ptr() if b is not None else 0 for c in self.caches
                        for b in (c.buffers() if hasattr(c, "buffers") else (c.keys,)))
        if buffers != self._buffers:                     # rings were (re)allocated: every captured pointer is stale
            self._graphs.clear()
            self._seen.clear()
            self._buffers = buffers
        if 0 in buffers:
            return None
        g = self._graphs.get(slots)
        if g is None:
            self._seen[slots] = self._seen.get(slots, 0) + 1
            if self._seen[slots] < 3:
                return None
            if len(self._graphs) >= 8:                   # a few live compositions at most: drop the oldest
                self._graphs.pop(next(iter(self._graphs)))
            g = self._graphs[slots] = _DecodeGraph(self, slots)
            self._seen.pop(slots, None)
        g.fill(tokens, pos0)
        return g.run(self)

    @torch.no_grad()
    def generate(self, prompts: Sequence[Sequence[int]], max_tokens: int = 64,
                 sampler: Optional[Callable[[torch.Tensor], torch.Tensor]] = None,
                 stop_tokens: Iterable[int] = ()) -> List[List[int]]:
        """Generate for several prompts at once: one ragged prompt step, then one token per live sequence and step.  A sequence that
        samples a stop token (or reaches ``max_tokens``) leaves the batch and frees its slot; the others go on.  ``sampler`` maps
        log-probabilities [n, vocab] to token ids [n] (default: greedy), as in ``generate_step``."""
        sampler = sampler or (lambda lp: torch.argmax(lp, dim=-1))
        stop = set(stop_tokens)
        ids = [object() for _ in prompts]
        out: List[List[int]] = [[] for _ in prompts]
        live = list(range(len(prompts)))
        feed = {i: list(prompts[i]) for i in live}
        while live:
            logits = self.step([(ids[i], feed[i]) for i in live])
            logprobs = logits - torch.logsumexp(logits, dim=-1, keepdim=True)
            toks = sampler(logprobs).reshape(-1).tolist()
            nxt = []
            for i, t in zip(live, toks):
                out[i].append(int(t))
                if int(t) in stop or len(out[i]) >= max_tokens:
                    self.release(ids[i])
                else:
                    feed[i] = [int(t)]
                    nxt.append(i)
            live = nxt
        return out
