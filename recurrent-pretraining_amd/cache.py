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


class _PositionView:
    """cache.key_cache[step]: positions -> [B, nh, hd] views into the contiguous storage."""

    def __init__(self, owner: "HuginnDynamicCache", store: str, step: int):
        self._o, self._store, self._step = owner, store, step

    def _filled(self) -> int:
        return self._o._filled.get(self._step, 0)

    def __len__(self):
        return self._filled()

    def __contains__(self, pos):
        return 0 <= int(pos) < self._filled()

    def __iter__(self):
        return iter(range(self._filled()))

    def keys(self):
        return range(self._filled())

    def values(self):
        return [self[p] for p in range(self._filled())]

    def items(self):
        return [(p, self[p]) for p in range(self._filled())]

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


class HuginnDynamicCache:
    """Drop-in for the reference class of the same name; storage is allocated on first use.

    `max_length` fixes the number of positions held (pointers then never move, which a captured HIP
    graph needs); without it the storage grows geometrically as tokens arrive.
    """

    def __init__(self, lookup_strategy: str = "full", max_length: Optional[int] = None):
        self._seen_tokens = 0
        self.lookup_strategy = lookup_strategy
        self.max_length = max_length
        self._k: Optional[torch.Tensor] = None
        self._v: Optional[torch.Tensor] = None
        self._neg_slots = 0          # slots reserved for negative (coda) step indices
        self._filled: dict[int, int] = {}  # step -> number of positions present (first-touch order)
        self.key_cache = _StepView(self, "_k")
        self.value_cache = _StepView(self, "_v")
        self._struct: Optional[hip.KVCache] = None

    # ---- storage ---------------------------------------------------------------------------
    def _slot(self, step: int) -> int:
        return self._neg_slots + step if step >= 0 else -step - 1

    @property
    def t_max(self) -> int:
        return 0 if self._k is None else self._k.shape[3]

    def ensure(self, n_pos_steps: int, n_neg_steps: int, batch: int, n_heads: int, head_dim: int, t_needed: int,
               dtype: torch.dtype, device) -> None:
        """Makes room for step indices -n_neg_steps .. n_pos_steps-1 and t_needed positions."""
        if self._k is not None:
            n_slots, b, nh, t_max, hd = self._k.shape
            if (b, nh, hd) != (batch, n_heads, head_dim) or self._k.dtype != dtype:
                raise ValueError(f"cache holds [B={b}, nh={nh}, hd={hd}] {self._k.dtype}; "
                                 f"asked for [B={batch}, nh={n_heads}, hd={head_dim}] {dtype}")
            if n_neg_steps <= self._neg_slots and n_pos_steps <= n_slots - self._neg_slots and t_needed <= t_max:
                return
            if self.max_length is not None and t_needed > self.max_length:
                raise ValueError(f"sequence of {t_needed} positions exceeds the cache's max_length {self.max_length}")
        if self.max_length is not None:
            if t_needed > self.max_length:
                raise ValueError(f"sequence of {t_needed} positions exceeds the cache's max_length {self.max_length}")
            new_t = self.max_length
        else:
            new_t = max(256, self.t_max)
            while new_t < t_needed:
                new_t *= 2
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

    def native(self) -> hip.KVCache:
        """The C-ABI descriptor of the storage (device pointers; rebuilt after every reallocation)."""
        if self._k is None:
            raise RuntimeError("cache storage has not been allocated yet")
        if self._struct is None:
            self._struct = hip.make_cache(self._k, self._v)
        return self._struct

    def note_append(self, step_idx: int, n_new: int, first_pos: int) -> int:
        """Bookkeeping for positions the kernels wrote at `step_idx`; returns the slot used."""
        step = remap_step(int(step_idx), self.lookup_strategy)
        if "compress-" not in self.lookup_strategy:  # RMM:192-193: no overwrite except for the coda
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
        lookup = self.lookup_strategy if lookup_strategy is None else lookup_strategy
        if self._filled[mapped] != self._seen_tokens and self.lookup_strategy != "full":
            raise NotImplementedError(f"lookup strategy {lookup!r} with positions missing at step {step}")
        t = self._filled[mapped]
        return self._k[slot, :, :, :t], self._v[slot, :, :, :t]

    def reset(self) -> None:  # RMM:275-279
        self._seen_tokens = 0
        self._filled.clear()

    def clear_last_k_entries(self, k: int = 0):  # RMM:281-293
        assert self._seen_tokens >= k
        self._seen_tokens -= k
        self._filled = {s: min(n, self._seen_tokens) for s, n in self._filled.items()}

    def get_seq_length(self, step_idx: int = 0) -> int:  # RMM:295-296
        return self._seen_tokens

    def get_memory_usage(self) -> float:
        """MiB held by the cached entries, counted as the reference does (key bytes doubled, RMM:298-308)."""
        if self._k is None:
            return 0.0
        _, b, nh, _, hd = self._k.shape
        per_pos = b * nh * hd * self._k.element_size()
        return sum(self._filled.values()) * per_pos * 2 / (1024 * 1024)

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
