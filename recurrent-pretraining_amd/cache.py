"""Step-indexed KV cache with the interface of the reference's HuginnDynamicCache
(recpre/raven_modeling_minimal.py:148-308) and the storage of its HuginnStaticCache (RMM:311-433):
two contiguous device tensors [n_slots, batch, n_heads, t_max, head_dim] that the HIP kernels
append to and read in place.  The reference keeps a dict cache[step][position] of small tensors and
re-stacks all of them on every block call; here `key_cache[step][pos]` is a view computed on demand.

Slots: the coda's negative step indices come first (step -1 -> slot 0, -2 -> slot 1, ...), the
non-negative ones follow (step s -> slot n_coda_slots + s), so a forward with more recurrences than
any earlier one only appends slots.
"""

from __future__ import annotations

import bisect
import math
from typing import Optional

import torch

from . import hip


def remap_step(step_idx: int, strategy: str) -> int:
    """Cache-sharing remap of the step index (RMM:169-182; hard-codes 2 prelude and 4 core blocks)."""
    if "compress-" in strategy and step_idx > 1:
        if "compress-s" in strategy:
            n = int(strategy.split("compress-")[1][1:])
            return (step_idx - 2) % n + 2
        if "compress-anchor" in strategy:
            return step_idx if step_idx - 2 < 32 else 34 + (step_idx - 34) % 4
        n = int(strategy.split("compress-")[1][1:])
        return (step_idx - 2) // n + 2
    return step_idx


class _CoreSteps:
    """Which core steps (step index 2, 3, ... = bit 0, 1, ...) are cached for which position, as runs
    [start, end, mask] of neighbouring positions with the same set: a prefill is one run, a decoded token
    joins the run before it when it was computed with the same number of recurrences."""

    def __init__(self):
        self.runs: list[list[int]] = []

    def __len__(self) -> int:
        return self.runs[-1][1] if self.runs else 0

    def _split(self, pos: int) -> int:
        """Index of the run that starts at pos (splitting the run that holds it); len(runs) when pos is the end."""
        i = bisect.bisect_right(self.runs, pos, key=lambda r: r[0]) - 1
        if i < 0 or pos >= self.runs[i][1]:
            return i + 1
        if self.runs[i][0] == pos:
            return i
        st, en, mask = self.runs[i]
        self.runs[i][1] = pos
        self.runs.insert(i + 1, [pos, en, mask])
        return i + 1

    def add(self, bit: int, first: int, n: int, overwrite: bool = False) -> None:
        """Positions first .. first+n-1 now hold core step `bit`; a second write of the same entry is an error unless
        the steps share entries (the compress-* strategies)."""
        if len(self) < first + n:
            self.runs.append([len(self), first + n, 0])
        i, j = self._split(first), self._split(first + n)
        for r in self.runs[i:j]:
            assert overwrite or not (r[2] >> bit) & 1, "overwrite of a cached position"  # RMM:192-193
            r[2] |= 1 << bit
        for k in range(min(j, len(self.runs) - 1), max(i - 1, 0) - 1, -1):  # re-join equal neighbours
            if k + 1 < len(self.runs) and self.runs[k][2] == self.runs[k + 1][2]:
                self.runs[k][1] = self.runs[k + 1][1]
                del self.runs[k + 1]

    def truncate(self, n: int) -> None:
        while self.runs and self.runs[-1][0] >= n:
            self.runs.pop()
        if self.runs:
            self.runs[-1][1] = min(self.runs[-1][1], n)

    def has(self, bit: int, pos: int) -> bool:
        i = bisect.bisect_right(self.runs, pos, key=lambda r: r[0]) - 1
        return i >= 0 and pos < self.runs[i][1] and bool((self.runs[i][2] >> bit) & 1)

    def count(self, bit: int, n: int) -> int:
        return sum(min(en, n) - st for st, en, mask in self.runs if st < n and (mask >> bit) & 1)

    @staticmethod
    def depth(mask: int) -> int:
        """Number of steps cached without a hole, from the first one on."""
        return (~mask & (mask + 1)).bit_length() - 1

    def min_depth(self, n: int) -> int:
        """Smallest depth over positions 0 .. n-1 (0 when some are unknown)."""
        if n > len(self):
            return 0
        return min((self.depth(mask) for st, en, mask in self.runs if st < n), default=0)

    def holes(self, n: int) -> bool:
        """True when a position below n holds a step but not all the steps before it."""
        return any(mask & (mask + 1) for st, en, mask in self.runs if st < n)

    def depths(self, n: int) -> list[int]:
        out: list[int] = []
        for st, en, mask in self.runs:
            if st < n:
                out.extend([self.depth(mask)] * (min(en, n) - st))
        return out


def lookup_mode(strategy: str) -> int:
    """What to do with positions that are not cached at the step being read (RMM:199-273)."""
    if strategy == "full" or strategy.startswith("skip"):
        return hip.LOOKUP_SKIP           # RMM:199-204 stacks whatever is there; RMM:247-254
    if strategy.startswith("latest-m4") or strategy.startswith("available-m4"):
        return hip.LOOKUP_LATEST         # RMM:206-232: the same for caches whose positions hold a prefix of the steps
    if strategy.startswith("always-last-m4"):
        return hip.LOOKUP_ALWAYS_LAST    # RMM:233-246
    if strategy.startswith("randomized"):
        # a sanity check in the reference (RMM:255-271): HuginnDynamicCache.update serves it on the host, one CPU draw
        # per position as there; the attention kernels, which resolve lookups in place, do not
        raise NotImplementedError("the 'randomized' lookup is served by HuginnDynamicCache.update only, not by the attention kernels")
    raise ValueError(f"Unknown lookup strategy: {strategy}")  # RMM:272-273


class _PositionView:
    """cache.key_cache[step]: positions -> [B, nh, hd] views into the contiguous storage."""

    def __init__(self, owner: "HuginnDynamicCache", store: str, step: int):
        self._o, self._store, self._step = owner, store, step

    def _positions(self):
        return [p for p in range(self._o._filled.get(self._step, 0)) if self._o._present(self._step, p)]

    def __len__(self):
        return self._o._n_present(self._step)

    def __contains__(self, pos):
        return self._o._present(self._step, int(pos))

    def __iter__(self):
        return iter(self._positions())

    def keys(self):
        return self._positions()

    def values(self):
        return [self[p] for p in self._positions()]

    def items(self):
        return [(p, self[p]) for p in self._positions()]

    def __getitem__(self, pos):
        if pos not in self:
            raise KeyError(pos)
        t = getattr(self._o, self._store)
        return t[self._o._slot(self._step), :, :, int(pos), :]


class _StepView:
    """cache.key_cache: step index -> _PositionView, in first-touch order like the reference's dict."""

    def __init__(self, owner: "HuginnDynamicCache", store: str):
        self._o, self._store = owner, store

    def __contains__(self, step):
        return int(step) in self._o._filled

    def __iter__(self):
        return iter(list(self._o._filled))

    def __len__(self):
        return len(self._o._filled)

    def keys(self):
        return list(self._o._filled)

    def items(self):
        return [(s, self[s]) for s in self._o._filled]

    def values(self):
        return [self[s] for s in self._o._filled]

    def __getitem__(self, step):
        if step not in self:
            raise KeyError(step)
        return _PositionView(self._o, self._store, int(step))


def line_aligned_positions(t: int, head_dim: int, dtype: torch.dtype) -> int:
    """The position capacity actually allocated for `t` positions: the next one at which a head's positions
    ([t_max, head_dim], contiguous) fill whole 128-byte cache lines.  With 192-byte rows (head_dim 96, bf16) an odd
    capacity puts every second head's rows 64 bytes into a line, and the decode attention kernel, which streams those
    rows, loses 7 % (32 sequences x 1024 positions: 115 us at a capacity of 1025, 107 us at 1026)."""
    row = head_dim * torch.empty((), dtype=dtype).element_size()
    unit = 128 // math.gcd(128, row)
    return (t + unit - 1) // unit * unit


class HuginnDynamicCache:
    """Drop-in for the reference class of the same name; storage is allocated on first use.

    `max_length` fixes the number of positions held (pointers then never move, which a captured HIP
    graph needs); without it the storage grows geometrically as tokens arrive.
    """

    is_compileable = False  # what transformers' generation loop asks a cache before it considers compiling the forward

    def __init__(self, lookup_strategy: str = "full", max_length: Optional[int] = None):
        self._seen_tokens = 0
        self.lookup_strategy = lookup_strategy
        self.max_length = max_length
        self._k: Optional[torch.Tensor] = None
        self._v: Optional[torch.Tensor] = None
        self._neg_slots = 0          # slots reserved for negative (coda) step indices
        self._filled: dict[int, int] = {}  # step -> 1 + highest position present (first-touch order)
        # Tokens computed with different numbers of recurrences leave gaps at the deeper core steps.  A token runs its
        # core steps in order, so for the kernels "how many of the steps 2, 3, 4, ... are cached" per position says it
        # all.  Under a compress-* remap the same holds for the shared entries: every one of the reference's remaps sends
        # the steps 2, 3, 4, ... of a token to entries 2, 3, 4, ... without skipping one (RMM:169-182), later steps
        # overwriting earlier ones.
        self._core = _CoreSteps()
        self._sp_dev: Optional[torch.Tensor] = None   # device copy of the per-position depths, built on demand
        self._sp_valid = 0                            # positions of _sp_dev that are up to date
        self._min_memo = (0, 0)                       # (n, smallest depth below n): older positions never change
        self._struct: Optional[hip.KVCache] = None

    # views made on access: a view stored on the cache would tie it into a reference cycle, and its tens of GB would
    # then stay allocated until the garbage collector happens to run
    @property
    def key_cache(self) -> _StepView:
        return _StepView(self, "_k")

    @property
    def value_cache(self) -> _StepView:
        return _StepView(self, "_v")

    # ---- storage ---------------------------------------------------------------------------
    def _slot(self, step: int) -> int:
        return self._neg_slots + step if step >= 0 else -step - 1

    @property
    def t_max(self) -> int:
        return 0 if self._k is None else self._k.shape[3]

    def ensure(self, n_pos_steps: int, n_neg_steps: int, batch: int, n_heads: int, head_dim: int, t_needed: int,
               dtype: torch.dtype, device) -> None:
        """Makes room for step indices -n_neg_steps .. n_pos_steps-1 and t_needed positions."""
        if self.max_length is not None and t_needed > self.max_length:  # the storage may hold a little more (whole cache lines)
            raise ValueError(f"sequence of {t_needed} positions exceeds the cache's max_length {self.max_length}")
        if self._k is not None:
            n_slots, b, nh, t_max, hd = self._k.shape
            if (b, nh, hd) != (batch, n_heads, head_dim) or self._k.dtype != dtype:
                raise ValueError(f"cache holds [B={b}, nh={nh}, hd={hd}] {self._k.dtype}; "
                                 f"asked for [B={batch}, nh={n_heads}, hd={head_dim}] {dtype}")
            if n_neg_steps <= self._neg_slots and n_pos_steps <= n_slots - self._neg_slots and t_needed <= t_max:
                return
        if self.max_length is not None:
            new_t = self.max_length
        else:
            new_t = max(256, self.t_max)
            while new_t < t_needed:
                new_t *= 2
        new_t = line_aligned_positions(new_t, head_dim, dtype)
        old_neg = self._neg_slots
        old_pos = 0 if self._k is None else self._k.shape[0] - old_neg
        new_neg, new_pos = max(old_neg, n_neg_steps), max(old_pos, n_pos_steps)
        shape = (new_neg + new_pos, batch, n_heads, new_t, head_dim)
        k = torch.zeros(shape, dtype=dtype, device=device)
        v = torch.zeros(shape, dtype=dtype, device=device)
        if self._k is not None:
            t_old = self._k.shape[3]
            for dst, src in ((k, self._k), (v, self._v)):
                dst[:old_neg, :, :, :t_old] = src[:old_neg]
                dst[new_neg:new_neg + old_pos, :, :, :t_old] = src[old_neg:]
        self._k, self._v, self._neg_slots = k, v, new_neg
        self._struct = None

    def native(self, steps=None, first_pos: int = 0) -> hip.KVCache:
        """The C-ABI descriptor of the storage (device pointers; rebuilt after every reallocation).

        With `steps` (the step indices a launch reads) and the first position of its new rows: the descriptor that
        makes the attention kernels resolve positions older than `first_pos` which are not cached at those steps
        according to the lookup strategy -- the plain one when there are no such gaps."""
        if self._k is None:
            raise RuntimeError("cache storage has not been allocated yet")
        if self._struct is None:
            self._struct = hip.make_cache(self._k, self._v)
        if steps is None or not any(self.has_gap(s, first_pos) for s in steps):
            return self._struct
        if not all(self.has_gap(s, first_pos) for s in steps):
            raise ValueError("steps of one launch must agree on whether older positions are missing")
        mode = lookup_mode(self.lookup_strategy)
        if mode == hip.LOOKUP_ALWAYS_LAST and "compress-" in self.lookup_strategy:
            # the reference then also looks up the new rows themselves, among entries their own earlier recurrences left
            raise NotImplementedError("always-last-m4 lookups over shared (compress-*) entries with missing positions are not built")
        if self._core.holes(first_pos):
            raise NotImplementedError("lookups need positions that hold the core steps 2, 3, ... without holes")
        if mode != hip.LOOKUP_SKIP and self._min_core(first_pos) <= max((remap_step(int(s), self.lookup_strategy) - 2) % 4 for s in steps):
            raise ValueError("a cached position holds no step to look up")  # the reference's max() of an empty list
        t_max = self.t_max
        if self._sp_dev is None or self._sp_dev.numel() < t_max:
            self._sp_dev, self._sp_valid = torch.zeros(t_max, dtype=torch.int32, device=self._k.device), 0
        if self._sp_valid < first_pos:
            self._sp_dev[:first_pos] = torch.tensor(self._core.depths(first_pos), dtype=torch.int32)
            self._sp_valid = first_pos
        return hip.make_cache(self._k, self._v, self._sp_dev, mode, self._slot(2))

    @staticmethod
    def _tracks_core(step: int) -> bool:
        return step >= 2

    def _present(self, step: int, pos: int) -> bool:
        if not 0 <= pos < self._filled.get(step, 0):
            return False
        return self._core.has(step - 2, pos) if self._tracks_core(step) else True

    def _n_present(self, step: int) -> int:
        n = self._filled.get(step, 0)
        return self._core.count(step - 2, n) if self._tracks_core(step) else n

    def has_gap(self, step_idx: int, first_pos: int) -> bool:
        """True when a position older than `first_pos` is not cached at this step."""
        step = remap_step(int(step_idx), self.lookup_strategy)
        if first_pos <= 0:
            return False
        if not self._tracks_core(step):
            return False  # the prelude and coda entries: every token passes through them
        return self._min_core(first_pos) <= step - 2

    def _min_core(self, n: int) -> int:
        if self._min_memo[0] != n:
            self._min_memo = (n, self._core.min_depth(n))
        return self._min_memo[1]

    def note_append(self, step_idx: int, n_new: int, first_pos: int) -> int:
        """Bookkeeping for positions the kernels wrote at `step_idx`; returns the slot used."""
        step = remap_step(int(step_idx), self.lookup_strategy)
        shared = "compress-" in self.lookup_strategy
        if self._tracks_core(step):
            self._core.add(step - 2, first_pos, n_new, overwrite=shared)
        elif not shared:  # RMM:192-193: no overwrite except for the coda
            assert step < 0 or self._filled.get(step, 0) <= first_pos, "overwrite of a cached position"
        self._filled[step] = max(self._filled.get(step, 0), first_pos + n_new)
        return self._slot(step)

    # ---- reference interface -----------------------------------------------------------------
    def update(self, key_states: torch.Tensor, value_states: torch.Tensor, step_idx_tensor,
               lookup_strategy: Optional[str] = None):
        """key/value_states [B, nh, S, hd] -> (K, V) [B, nh, T, hd] of that step (RMM:160-204).

        For callers that drive the cache themselves with torch tensors; the model's own forward
        lets the kernels write the storage directly and only does the bookkeeping."""
        step = int(step_idx_tensor)
        b, nh, n_new, hd = key_states.shape
        mapped = remap_step(step, self.lookup_strategy)
        if mapped == 0:  # RMM:188-189
            self._seen_tokens += n_new
        first = self._seen_tokens - n_new
        self.ensure(max(mapped + 1, 1), max(-mapped, 0), b, nh, hd, self._seen_tokens, key_states.dtype, key_states.device)
        slot = self.note_append(step, n_new, first)
        self._k[slot, :, :, first:first + n_new] = key_states
        self._v[slot, :, :, first:first + n_new] = value_states
        if self._n_present(mapped) == self._seen_tokens:
            return self._k[slot, :, :, :self._seen_tokens], self._v[slot, :, :, :self._seen_tokens]
        # some positions were never computed at this step: gather per position, as RMM:199-253 does
        lookup = self.lookup_strategy if lookup_strategy is None else lookup_strategy
        if self.lookup_strategy != "full" and lookup.startswith("randomized"):
            return self._gather_randomized(mapped)
        mode = hip.LOOKUP_SKIP if self.lookup_strategy == "full" else lookup_mode(lookup)
        if mode == hip.LOOKUP_ALWAYS_LAST and "compress-" in self.lookup_strategy:
            raise NotImplementedError("always-last-m4 lookups over shared (compress-*) entries with missing positions are not built")
        if self._core.holes(first):
            raise NotImplementedError("lookups need positions that hold the core steps 2, 3, ... without holes")
        depths = self._core.depths(first) if self._tracks_core(mapped) else []
        src = [self._source_step(mapped, depths[p], mode) if p < len(depths) else mapped for p in range(self._seen_tokens)]
        pos = torch.tensor([p for p, st in enumerate(src) if st is not None], device=self._k.device)
        slots = torch.tensor([self._slot(st) for st in src if st is not None], device=self._k.device)
        return self._k[slots, :, :, pos].permute(1, 2, 0, 3), self._v[slots, :, :, pos].permute(1, 2, 0, 3)

    def _gather_randomized(self, step: int):
        """RMM:255-271: every position, the new ones included, is read at a step drawn among those of the same block
        that it holds up to `step` -- one `torch.randint` on the CPU's default generator per position, in position
        order, as the reference draws them (an empty choice raises there and here)."""
        if self._core.holes(self._seen_tokens):
            raise NotImplementedError("lookups need positions that hold the core steps 2, 3, ... without holes")
        src = []
        for depth in self._core.depths(self._seen_tokens):
            valid = [s for s in range(2, step + 1) if (s - step) % 4 == 0 and s - 2 < depth]
            src.append(valid[int(torch.randint(len(valid), (1,)))])
        pos = torch.arange(self._seen_tokens, device=self._k.device)
        slots = torch.tensor([self._slot(st) for st in src], device=self._k.device)
        return self._k[slots, :, :, pos].permute(1, 2, 0, 3), self._v[slots, :, :, pos].permute(1, 2, 0, 3)

    @staticmethod
    def _source_step(step: int, depth: int, mode: int):
        """The step whose entry stands in for `step` (>= 2) at a position of an earlier token that holds `depth` core
        steps, or None when the position is left out: what the attention kernels compute from steps_present."""
        cs = step - 2
        if mode != hip.LOOKUP_ALWAYS_LAST and cs < depth:
            return step
        if mode == hip.LOOKUP_SKIP:
            return None
        j = cs % 4
        if depth - 1 - j < 0:
            raise ValueError("a cached position holds no complete recurrence to look up")
        return 2 + j + (depth - 1 - j) // 4 * 4

    def reset(self) -> None:  # RMM:275-279
        self._seen_tokens = 0
        self._filled.clear()
        self._core = _CoreSteps()
        self._sp_valid = 0
        self._min_memo = (0, 0)

    def clear_last_k_entries(self, k: int = 0):  # RMM:281-293
        assert self._seen_tokens >= k
        self._seen_tokens -= k
        self._filled = {s: min(n, self._seen_tokens) for s, n in self._filled.items()}
        self._core.truncate(self._seen_tokens)
        self._sp_valid = min(self._sp_valid, self._seen_tokens)
        self._min_memo = (0, 0)

    def get_seq_length(self, step_idx: int = 0) -> int:  # RMM:295-296
        return self._seen_tokens

    def get_memory_usage(self) -> float:
        """MiB held by the cached entries, counted as the reference does (key bytes doubled, RMM:298-308)."""
        if self._k is None:
            return 0.0
        _, b, nh, _, hd = self._k.shape
        per_pos = b * nh * hd * self._k.element_size()
        return sum(self._n_present(s) for s in self._filled) * per_pos * 2 / (1024 * 1024)

    def get_allocated_mb(self) -> float:
        """MiB actually allocated (what HuginnStaticCache.get_memory_usage reports, RMM:432-433)."""
        if self._k is None:
            return 0.0
        return 2 * self._k.nelement() * self._k.element_size() / (1024 * 1024)


class HuginnStaticCache(HuginnDynamicCache):
    """The reference's preallocated cache (RMM:311-433) with its constructor signature.  Storage and
    behaviour are those of HuginnDynamicCache with `max_length` fixed; `max_num_steps` (= 4 + 4 * recurrences in
    the reference's callers) only presizes the slots."""

    def __init__(self, max_length: int, max_num_steps: int, num_heads: int, hidden_dim: int, batch_size: int = 1,
                 lookup_strategy: str = "full", device=None, dtype: torch.dtype = torch.float32) -> None:
        super().__init__(lookup_strategy=lookup_strategy, max_length=max_length)
        if "compress-" in lookup_strategy:  # RMM:330-338
            stage = int(lookup_strategy.split("compress-")[1][1:])
            steps = 4 + stage if "compress-s" in lookup_strategy else 4 + (max_num_steps - 4 + stage - 1) // stage
        else:
            steps = max_num_steps
        self.max_num_steps = steps
        n_neg = 2 if steps >= 4 else 1
        self.ensure(max(steps - n_neg, 1), n_neg, batch_size, num_heads, hidden_dim, max_length, dtype,
                    device if device is not None else "cpu")

    def get_memory_usage(self) -> float:
        """Allocated MiB, as the reference's static cache reports (RMM:432-433)."""
        return self.get_allocated_mb()
