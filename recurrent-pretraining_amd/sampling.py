"""Logit penalties applied before a token is picked (recpre/raven_modeling_minimal.py:1991-2070): the standard
repetition penalty over the tokens seen so far, and the n-gram ("DRY") penalty that is selected by a positive
`dry_multiplier` in the generation settings.  Plain tensor code: a few thousand elements per generated token."""

from __future__ import annotations

import torch


def _dry_penalties(context: list, multiplier: float, base: float, allowed_length: int) -> dict:
    """token -> penalty for continuing a repetition.  For every start in the last 128 positions, the run that matches
    the reversed tail of the context (at most 32 long) is measured as the reference measures it; the token that
    follows the run would extend it to run + 1, and a token is penalised by its longest such extension."""
    n = len(context)
    longest: dict = {}
    for start in range(max(0, n - 128), n - 1):
        run = 0
        while start + run < n and run < 32 and context[start + run] == context[n - run - 1]:
            run += 1
        if run > 0 and start + run < n:
            tok = context[start + run]
            if run + 1 > longest.get(tok, 0):
                longest[tok] = run + 1
    return {tok: multiplier * base ** (m - allowed_length) for tok, m in longest.items() if m >= allowed_length}


def apply_repetition_penalty(original_logits: torch.Tensor, input_ids: torch.Tensor, generation_config, use_candidates: bool = False):
    """RMM:1991-2070.  original_logits [B, V], [T, V] (one sequence, several positions) or [B, T, V]; returns float32
    logits of the same shape.  use_candidates appends the positions' own argmax tokens to the context."""
    if original_logits.dim() == 2:
        per_batch = original_logits.shape[0] == input_ids.shape[0]
        logits = original_logits.unsqueeze(1 if per_batch else 0).to(copy=True, dtype=torch.float32)
    else:
        logits = original_logits.clone()
    B, T, V = logits.shape
    dry = getattr(generation_config, "dry_multiplier", 0) or 0
    if dry > 0:
        base = getattr(generation_config, "dry_base", 1.75)
        allowed = getattr(generation_config, "dry_allowed_length", 2)
        for b in range(B):
            context = input_ids[b].tolist()
            if use_candidates:
                context = context + logits[b].argmax(dim=-1).tolist()
            pen = _dry_penalties(context, dry, base, allowed)  # the same for every position of the row, as in the reference
            if pen:
                idx = torch.tensor([t for t in pen if 0 <= t < V], device=logits.device, dtype=torch.long)
                val = torch.tensor([pen[int(t)] for t in idx.tolist()], device=logits.device, dtype=logits.dtype)
                logits[b, :, idx] -= val
    else:
        penalty = generation_config.repetition_penalty
        for b in range(B):
            sequence = input_ids[b]
            if use_candidates:
                sequence = torch.cat([sequence, logits[b].argmax(dim=-1)])
            seen = torch.unique(sequence)
            picked = logits[b][:, seen]
            logits[b][:, seen] = torch.where(picked < 0, picked * penalty, picked / penalty)
    if original_logits.dim() == 2:
        return logits.squeeze(1 if per_batch else 0)
    return logits
