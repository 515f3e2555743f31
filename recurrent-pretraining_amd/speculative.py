"""Self-speculative decoding (recpre/raven_modeling_minimal.py:1750-1927): the model drafts a few tokens with a
small number of recurrences, drops them from the cache, and verifies all of them in one forward with the full
number of recurrences -- a chunk of `lookahead_for_draft` rows through the same kernels a prefill uses.

The loop is the reference's, tensor operation by tensor operation (including what it does to batches: sequences
that accept fewer tokens are padded with `pad_id` and the cache is rolled back to the shortest accepted prefix; once
the sequences of a batch have accepted different numbers of tokens the loop goes on, as the reference's does, with
RoPE positions that differ from the cache positions -- forward() rotates by the positions it is given)."""

from __future__ import annotations

from typing import Callable, Optional

import torch


@torch.no_grad()
def generate_speculative(model, input_ids: torch.Tensor, generation_config=None, tokenizer=None, streamer=None,
                         continuous_compute: bool = False, init_scale: float = 1.0, cache_lookup_strategy: str = "full",
                         draft_steps: int = 32, lookahead_for_draft: int = 8, verification_threshold=1, num_steps: int = 32,
                         input_states_fn: Optional[Callable] = None, stop_tokens: Optional[set] = None, pad_id: int = 65509,
                         **model_kwargs):
    """RMM:1750-1927.  Extensions: input_states_fn(call, (B, S, h)) supplies the initial latent state of the call-th
    forward (prefill, drafts and verifications counted in order; call -1 is the warm-start state of continuous
    compute); stop_tokens overrides the reference's fixed stop set; pad_id (the reference hard-codes 65509) fills the
    rows of sequences that accepted fewer tokens than others; with return_dict_in_generate the output's
    `scores` carries "accepted_tokens" per round and sequence."""
    from .modeling import GenerateOutput

    assert lookahead_for_draft > 0
    L = lookahead_for_draft
    gc = generation_config if generation_config is not None else model.generation_config
    B, prompt_len = input_ids.shape
    if model_kwargs.get("max_new_tokens") is not None:
        max_new = model_kwargs["max_new_tokens"]
        if "max_length" in model_kwargs:
            max_new = min(max_new, model_kwargs["max_length"] - prompt_len)
    elif getattr(gc, "max_new_tokens", None):
        max_new = gc.max_new_tokens
    else:
        max_new = model_kwargs.get("max_length", model._default_max_length(gc)) - prompt_len
    stops = model._get_stops(gc) if stop_tokens is None else set(stop_tokens)
    dev, h = model.device, model.config.n_embd
    input_ids = input_ids.to(dev)
    cache = model._generation_cache(model_kwargs, cache_lookup_strategy, B)
    calls = [0]

    def run(tokens, pos, steps, carried):
        state = carried
        if state is None and input_states_fn is not None:
            state = input_states_fn(calls[0], (B, tokens.shape[1], h)).to(dev, model.dtype)
        calls[0] += 1
        return model.forward(input_ids=tokens.contiguous(), input_states=state, num_steps=steps, past_key_values=cache,
                             use_cache=True, cache_position=pos, init_scale=init_scale)

    carried = None
    if continuous_compute:
        if input_states_fn is not None:
            carried = input_states_fn(-1, (B, prompt_len, h)).to(dev, model.dtype)
        else:
            carried = model.initialize_state(model.embed_inputs(input_ids)[0], scale=init_scale)
    unfinished = torch.ones(B, dtype=torch.bool)
    generated = 0
    if cache.get_seq_length() == 0:  # prefill with the full number of steps
        out = run(input_ids, torch.arange(0, prompt_len, device=dev), num_steps, carried)
        next_token = model._sample_next_token(out.logits[:, -1, :], input_ids, gc)
        input_ids = torch.cat([input_ids, next_token], dim=-1)
        generated += 1
        if streamer:
            streamer.put(next_token.cpu())
        if continuous_compute:
            carried = out.latent_states[:, -1:, :]
    cache_position = torch.tensor([cache.get_seq_length()], device=dev)
    prefix_len = input_ids.shape[1]
    accepted_tokens = []

    while generated < max_new:
        drafted = input_ids.clone()
        current_len = input_ids.shape[1]
        for _ in range(L):
            out = run(drafted[:, cache_position], cache_position, draft_steps, carried)
            next_token = model._sample_next_token(out.logits[:, -1, :], drafted, gc)
            drafted = torch.cat([drafted, next_token], dim=-1)
            cache_position = cache_position[-1:] + 1
            if continuous_compute:
                carried = out.latent_states[:, -1:, :]
        cache.clear_last_k_entries(L)

        cache_position = torch.arange(current_len - 1, current_len + L - 1, device=dev)
        out = run(drafted[:, cache_position], cache_position, num_steps, carried)
        preds = out.logits.argmax(dim=-1)
        if verification_threshold >= 1:
            mismatched = preds[:, -L:] != drafted[:, current_len:]
            not_all, first_mismatch = torch.max(mismatched, dim=1)
        else:
            probs = torch.softmax(out.logits[:, -L:, :], dim=-1)
            drafted_p = torch.gather(probs, -1, drafted[:, current_len:].unsqueeze(-1)).squeeze(-1)
            passed = drafted_p >= verification_threshold * probs.max(dim=-1)[0]
            not_all, first_mismatch = torch.max(~passed, dim=1)
        accept = torch.where(not_all, first_mismatch, L).tolist()
        not_all_l = not_all.tolist()
        per_seq = []
        for i in range(B):
            a = accept[i]
            if not_all_l[i] and a < L:  # accept up to the mismatch, then the verifier's own token
                final = model._sample_next_token(out.logits[i:i + 1, a, :], input_ids, gc)
                part = drafted[i:i + 1, current_len:current_len + a]
                per_seq.append(torch.cat([part, final], dim=-1) if a > 0 else final)
            else:
                per_seq.append(drafted[i:i + 1, current_len:current_len + a])
        if any(not_all_l):
            cache.clear_last_k_entries(L - int(first_mismatch.min()) - 1)
        counts = [t.shape[1] for t in per_seq]
        width = max(counts)
        rows = [torch.cat([t, pad_id * torch.ones((1, width - t.shape[1]), dtype=t.dtype, device=dev)], dim=-1)
                if t.shape[1] < width else t for t in per_seq]
        input_ids = torch.cat([input_ids, torch.cat(rows, dim=0)], dim=-1)
        accepted_tokens.append(counts)
        generated += width
        if streamer:
            streamer.put(per_seq[0].cpu())
        cache_position = torch.tensor([cache.get_seq_length()], device=dev)
        if continuous_compute:
            carried = out.latent_states[:, -1:, :]
        if stops:
            for i in range(B):
                if unfinished[i] and any(t in stops for t in per_seq[i].flatten().tolist()):
                    unfinished[i] = False
        if "stopping_criteria" in model_kwargs:
            unfinished = unfinished & ~model_kwargs["stopping_criteria"](input_ids, None).cpu()
        if not bool(unfinished.any()):
            break
    if streamer:
        streamer.end()
    if stops:  # cut each sequence after its first stop token
        for i in range(B):
            hits = [j for j, t in enumerate(input_ids[i, prefix_len:].tolist()) if t in stops]
            if hits:
                input_ids[i, prefix_len + hits[0] + 1:] = pad_id
    real = (input_ids != pad_id).any(dim=0).nonzero()
    if len(real) > 0:
        input_ids = input_ids[:, :int(real[-1]) + 1]
    if getattr(gc, "return_dict_in_generate", False):
        return GenerateOutput(sequences=input_ids, past_key_values=cache, scores={"accepted_tokens": accepted_tokens})
    return input_ids
