"""
Slot state manager for models whose per-sequence memory is bounded: every sequence that is alive holds one SLOT, and a slot holds, for
each layer, what that layer's mixer declares -- a ring buffer of the last `window` keys and values for sliding-window attention, a
float32 matrix per head for a recurrent (linear-attention) layer.  Slots are handed out on admission, given back when a sequence ends
and used again by the next one; the pool grows by doubling when every slot is taken.  Nothing in a slot has to be cleared on reuse: a
mixer starts a sequence (position 0) from its own initial state and reads only what the sequence's length says is valid.

`StepBatch` describes one step of the engine over these slots: the packed rows of all sequences in the step, and where each sequence
stands.  The generator's scheduler and the trace runner both build it through `SlotStateCache.begin_step`.
"""
from __future__ import annotations
from dataclasses import dataclass, field
import torch


@dataclass
class StateSpec:
    """One per-slot buffer of a layer: name, shape per slot, element type."""
    name: str
    shape: tuple
    dtype: torch.dtype


@dataclass
class StepBatch:
    n: int                      # rows in the step
    batch: int                  # sequences in the step
    decode: bool                # every sequence brings exactly one row (mixers read their caches); otherwise every sequence starts at position 0
    max_rows: int               # longest sequence of the step
    tokens: torch.Tensor        # int32 [n]
    cu: torch.Tensor            # int32 [batch + 1], first row of each sequence
    tok_seq: torch.Tensor       # int32 [n]
    tok_pos: torch.Tensor       # int32 [n]
    slots: torch.Tensor         # int32 [batch]
    pos0: torch.Tensor          # int32 [batch], length before the step
    len_after: torch.Tensor     # int32 [batch], length after the step
    want_rows: torch.Tensor | None = None     # int32 [m]: rows whose logits are asked for (may be empty)
    host_lens: list = field(default_factory=list)
    buffer: torch.Tensor | None = None        # the one device array that the tensors above are views of


class SlotStateCache:
    def __init__(self, layer_specs: list[list[StateSpec]], device, slots: int = 4):
        self.device = torch.device(device)
        self.layer_specs = layer_specs
        self.capacity = 0
        self.layers: list[dict[str, torch.Tensor]] = [dict() for _ in layer_specs]
        self.free: list[int] = []
        self.length: dict[int, int] = {}         # slot -> tokens held by the sequence that owns it
        self.generation = 0
        self._grow(max(1, slots))

    def bytes_per_slot(self) -> int:
        total = 0
        for specs in self.layer_specs:
            for s in specs:
                nel = 1
                for d in s.shape:
                    nel *= d
                total += nel * torch.empty((), dtype=s.dtype).element_size()
        return total

    def _grow(self, new_capacity: int):
        for li, specs in enumerate(self.layer_specs):
            for s in specs:
                buf = torch.zeros((new_capacity,) + tuple(s.shape), dtype=s.dtype, device=self.device)
                old = self.layers[li].get(s.name)
                if old is not None:
                    buf[: self.capacity].copy_(old)
                self.layers[li][s.name] = buf
        self.free.extend(range(new_capacity - 1, self.capacity - 1, -1))      # lowest number on top of the stack
        self.capacity = new_capacity
        self.generation += 1                   # the buffers moved: whoever holds their addresses (captured graphs) starts over

    def alloc(self) -> int:
        if not self.free:
            self._grow(self.capacity * 2)
        slot = self.free.pop()
        self.length[slot] = 0
        return slot

    def release(self, slot: int):
        if slot not in self.length:
            raise RuntimeError(f"slot {slot} is not in use")
        del self.length[slot]
        self.free.append(slot)

    def in_use(self) -> int:
        return len(self.length)

    def begin_step(self, entries: list[tuple[int, list[int]]], want: list[list[int]] | None = None, into: StepBatch | None = None) -> StepBatch:
        """entries: (slot, the sequence's next tokens).  Either every sequence is at position 0 (a prompt step) or every sequence brings one
        token (a decode step).  want: per entry, the places among its tokens whose logits are asked for (None: every sequence's last).
        into: a StepBatch of the same layout (same row and sequence counts) whose device buffer is overwritten in place -- a captured graph keeps
        reading the same addresses."""
        lens = [len(t) for _, t in entries]
        if not entries or min(lens) < 1:
            raise RuntimeError("a step needs at least one token per sequence")
        pos0 = [self.length[s] for s, _ in entries]
        decode = all(l == 1 for l in lens) and any(p > 0 for p in pos0)
        if not decode and any(p > 0 for p in pos0):
            raise RuntimeError("a step either starts all its sequences or continues all of them by one token")
        n, b = sum(lens), len(entries)
        cu = [0]
        for l in lens:
            cu.append(cu[-1] + l)
        tokens, tok_seq, tok_pos = [], [], []
        for i, (_, t) in enumerate(entries):
            tokens.extend(t)
            tok_seq.extend([i] * len(t))
            tok_pos.extend(range(pos0[i], pos0[i] + len(t)))
        slots = [s for s, _ in entries]
        after = [p + l for p, l in zip(pos0, lens)]
        if want is None:
            rows = [c - 1 for c in cu[1:]]
        else:
            rows = [cu[i] + p for i, w in enumerate(want) for p in w]
        # one host array, one copy: the pieces are views of it on the device
        flat = tokens + cu + tok_seq + tok_pos + slots + pos0 + after + rows
        host = torch.tensor(flat, dtype=torch.int32)
        if into is not None:
            if (into.n, into.batch, into.decode, into.want_rows.numel()) != (n, b, decode, len(rows)) or into.buffer.numel() != len(flat):
                raise RuntimeError("begin_step(into=...): the step has another layout than the one the buffer was made for")
            into.buffer.copy_(host)
            for (s, _), a in zip(entries, after):
                self.length[s] = a
            into.host_lens = lens
            return into
        dev = host.to(self.device, non_blocking=False)
        cuts, at = [], 0
        for ln in (n, b + 1, n, n, b, b, b, len(rows)):
            cuts.append(dev[at: at + ln]); at += ln
        for (s, _), a in zip(entries, after):
            self.length[s] = a
        return StepBatch(n=n, batch=b, decode=decode, max_rows=max(lens), tokens=cuts[0], cu=cuts[1], tok_seq=cuts[2], tok_pos=cuts[3], slots=cuts[4],
                         pos0=cuts[5], len_after=cuts[6], want_rows=cuts[7], host_lens=lens, buffer=dev)
