"""Diffusion-style sampler (recpre/raven_modeling_minimal.py:1234-1549): instead of finishing one token after the other
with all recurrences, a wave of not-yet-frozen positions is advanced together by a few recurrences per step.  After
every step the wave's cache entries are dropped again (`clear_last_k_entries`), the tokens guessed for its positions
are updated from the new logits, `headway` new positions join at the right, and positions freeze from the left once
their latent state has stopped moving (or their token has been stable, or after a fixed number of steps).  Frozen
positions keep their keys and values; the cache strategy `latest-m4-compress-s4` lets every recurrence overwrite the
same four core slots, so a frozen position holds the entries of its last recurrence.

On the device this is the multi-row path: a step is one chunk of `wave` rows through the prelude, `inner_recurrence`
calls of the recurrent block, the coda and the head (forward's kernels: chunk attention over the cache, skinny or
library GEMMs by row count); the freezing criterion for `latent-diff` is the latent-statistics kernel of the
adaptive-compute loop.  The host loop is the reference's, statement by statement; one sequence per call, as there."""

from __future__ import annotations

from typing import Callable, Optional

import torch

from . import hip


@torch.no_grad()
def generate_diffusion_style(model, input_ids: torch.Tensor, generation_config=None, tokenizer=None, streamer=None,
                             init_scale: float = 1.0, cache_lookup_strategy: str = "latest-m4-compress-s4",
                             full_prefill: bool = True, ema_embeds: float = 0.1, state_noise_mixing: float = 0.5,
                             inner_recurrence: int = 4, num_steps: int = 32, freeze_strategy: str = "latent-diff",
                             headway: int = 1, dampened_state_mixer: bool = True, sqrt_mixer: bool = False,
                             continuous_compute: bool = False, exit_t: float = 0.03, max_wavefront: int = 128,
                             max_diffusion_steps: int = 4096, return_analysis_tablets: bool = False,
                             input_states_fn: Optional[Callable] = None, extra_tokens_fn: Optional[Callable] = None,
                             extra_token_high: int = 65510, stop_tokens: Optional[set] = None, **model_kwargs):
    """RMM:1234-1549.  Extensions: input_states_fn(draw, shape) supplies the draw-th random latent state (the prefill's
    initial state, the first wave state, then per step the noise states and the states of the new positions, in that
    order); extra_tokens_fn(step, n) the n = headway - 1 filler tokens of a step (the reference draws them below the
    hard-coded 65510, here `extra_token_high`); stop_tokens overrides the reference's stop set.  With
    return_dict_in_generate the output's `scores` holds the reference's summary (passes, tokens forwarded, cache
    clears, standing waves, steps, recurrences and stable steps per position)."""
    from .modeling import GenerateOutput

    if input_ids.shape[0] != 1:
        raise NotImplementedError("the diffusion-style sampler takes one sequence (so does the reference)")
    if return_analysis_tablets:
        raise NotImplementedError("analysis tablets are not recorded")
    gc = generation_config if generation_config is not None else model.generation_config
    cfg = model.config
    dev, dt, h = model.device, model.dtype, cfg.n_embd
    input_ids = input_ids.to(dev)
    n_prompt = input_ids.shape[1]
    if model_kwargs.get("max_new_tokens") is not None:
        max_new = model_kwargs["max_new_tokens"]
        if "max_length" in model_kwargs:
            max_new = min(max_new, model_kwargs["max_length"] - n_prompt)
    elif getattr(gc, "max_new_tokens", None):
        max_new = gc.max_new_tokens
    else:
        max_new = model_kwargs.get("max_length", model._default_max_length(gc)) - n_prompt
    stops = model._get_stops(gc) if stop_tokens is None else set(stop_tokens)
    cache = model._generation_cache(model_kwargs, cache_lookup_strategy, 1)
    draws = [0]

    def draw(shape, via_bf16: bool = False):
        """One random latent state (RMM:804-813); new positions come from a bf16 template in the reference."""
        if input_states_fn is not None:
            x = input_states_fn(draws[0], shape).to(dev)
        else:
            x = model.initialize_state(torch.empty(shape, device=dev, dtype=torch.bfloat16 if via_bf16 else dt), scale=init_scale)
        draws[0] += 1
        return (x.to(torch.bfloat16) if via_bf16 else x).to(dt)

    width = max(cfg.block_size, n_prompt + max_new + headway + int(full_prefill))
    rec_count = torch.zeros(1, width, dtype=torch.long)   # host side: only its values steer the loop
    stable = torch.zeros(1, width, dtype=torch.long)
    passes = tokens_forward = clears = standing = 0

    if full_prefill:
        out = model.forward(input_ids=input_ids, input_states=draw((1, n_prompt, h)), num_steps=num_steps, past_key_values=cache,
                            use_cache=True, cache_position=torch.arange(n_prompt, device=dev), init_scale=init_scale)
        passes, tokens_forward = passes + 1, tokens_forward + n_prompt
        next_token = model._sample_next_token(out.logits[:, -1, :], input_ids, gc)
        if streamer:
            streamer.put(next_token.cpu())
        frozen = current = torch.cat([input_ids, next_token], dim=-1)
        rec_count[:, :frozen.shape[1]] += num_steps
        states = draw((1, 1, h))
    else:
        states = draw((1, n_prompt, h), via_bf16=True)
        frozen, current = input_ids.clone(), input_ids.clone()
        if 0 < max_wavefront < states.shape[1]:
            raise ValueError("The input prompt is too long to fit into the chosen max_wavefront memory limit. Use prefill, "
                             f"or increase max_wavefront to at least {states.shape[1]}")

    if ema_embeds > 0.0:
        old_embeds, _ = model.embed_inputs(current)  # over the whole sequence, without a cache
    latent = "latent" in freeze_strategy
    accel = "latent-acceleration" in freeze_strategy
    if latent:
        prev_states = states.clone()
    if accel:
        prev_delta, prev_prev_states, old_old_ci = torch.zeros_like(states), torch.zeros_like(states), 0
    old_ci, old_k, k, step = 0, 0, 0, 0

    while frozen.shape[1] - n_prompt < max_new and current.shape[1] <= cfg.block_size:
        ci = cache.get_seq_length()
        n_wave = states.shape[1]
        pos = torch.arange(ci, ci + n_wave, device=dev)
        aux = dict(past_key_values=cache, cache_position=pos)
        new_embeds, block_idx = model.embed_inputs(current[:, ci:ci + n_wave].contiguous(), use_cache=True, **aux)
        if ema_embeds > 0.0:
            carry = old_embeds[:, ci - old_ci:]
            embeds = new_embeds.clone() * (1 - ema_embeds)
            embeds[:, :carry.shape[1], :] += carry * ema_embeds
            old_embeds = embeds.clone()
        else:
            embeds = new_embeds
        if state_noise_mixing > 0:
            noise_states = draw(tuple(states.shape))
            if dampened_state_mixer:
                mix = (state_noise_mixing / (1 + rec_count[:, ci:ci + n_wave]))[:, :, None].to(device=dev, dtype=dt)
            else:
                mix = torch.as_tensor(state_noise_mixing, device=dev, dtype=dt)
            if sqrt_mixer:
                states = states * torch.relu(1 - mix).sqrt() + mix.sqrt() * noise_states
            else:
                states = states * (1 - mix) + mix * noise_states
        for _ in range(inner_recurrence):
            states, block_idx, _ = model.iterate_one_step(embeds, states, block_idx=block_idx, **aux)
            rec_count[:, ci:ci + n_wave] += 1
            passes, tokens_forward = passes + 1, tokens_forward + n_wave
        logits = model.predict_from_latents(states, **aux).logits
        final_logits = logits[0, max(frozen.shape[1] - 1 - ci, 0):, :]
        new_tokens = model._sample_next_token(final_logits, frozen, gc).T
        guess = torch.cat([frozen, new_tokens[:, :-1]], dim=1)
        stable[:, :current.shape[1]] += (current == guess).cpu()
        if extra_tokens_fn is not None:
            extra = extra_tokens_fn(step, headway - 1).view(1, headway - 1).to(dev)
        else:
            extra = torch.randint(0, extra_token_high, (1, headway - 1), device=dev)
        current = torch.cat([frozen, new_tokens, extra], dim=1)
        if continuous_compute and states.shape[1] >= headway:
            fresh = states[:, -headway:].clone()
        else:
            fresh = draw((1, headway, h), via_bf16=True)
        states = torch.cat([states, fresh], dim=1)
        headway_now = headway
        if max_wavefront > 0 and states.shape[1] > max_wavefront:
            headway_now = max_wavefront - (states.shape[1] - headway)
            states = states[:, :max_wavefront]
            current = current[:, :ci + max_wavefront]
            standing += 1

        def freeze_up_to(k_new: int):
            """Positions < k_new are final: keep their cache entries, drop the rest of the wave's (RMM:1437-1444)."""
            nonlocal states, frozen, clears
            n_clear = current.shape[1] - headway_now - k_new + 1
            cache.clear_last_k_entries(n_clear)
            clears += n_clear
            states = states[:, k_new - ci - 1:, :]
            frozen = current[:, :k_new]
            if streamer:
                streamer.put(frozen[:, old_k:k_new].cpu())

        def freeze_nothing():
            nonlocal clears
            cache.clear_last_k_entries(states.shape[1] - headway_now)
            clears += states.shape[1] - headway_now

        if latent:
            if freeze_strategy == "latent-diff":
                old = prev_states[:, ci - old_ci:]
                cur = states[:, :old.shape[1], :]
                m = cur.shape[1]
                # |cur - old| / |cur| per position, with the reference's rounding points (the adaptive loop's kernel)
                criterion = hip.exit_latent_stats(cur.reshape(m, h).contiguous(), old.reshape(m, h).contiguous())[0].view(1, m)
            elif freeze_strategy == "latent-acceleration-1":
                old = prev_states[:, ci - old_ci:]
                cur = states[:, :old.shape[1], :]
                delta = cur - old
                m = min(delta.shape[1], prev_delta.shape[1])
                criterion = (delta[:, :m, :] - prev_delta[:, :m, :]).norm(dim=-1) / cur[:, :m, :].norm(dim=-1)
                prev_delta = delta.clone()
            elif freeze_strategy == "latent-acceleration-2":
                lo = max(ci, old_ci, old_old_ci)
                hi = min(ci + states.shape[1], old_ci + prev_states.shape[1], old_old_ci + prev_prev_states.shape[1])
                a, b, c = (states[:, lo - ci:hi - ci], prev_states[:, lo - old_ci:hi - old_ci],
                           prev_prev_states[:, lo - old_old_ci:hi - old_old_ci])
                criterion = ((a - b) - (b - c)).norm(dim=-1) / (a.norm(dim=-1) + 1e-6)
            else:
                raise ValueError(f"Invalid freeze strategy {freeze_strategy}")
            exits = [i for i, e in enumerate((criterion < exit_t)[0].tolist()) if e]  # one device-to-host read per step
            if exits:
                k = ci + exits[-1] + 1
                freeze_up_to(k)
            else:
                freeze_nothing()
        elif freeze_strategy == "token-stability":
            ripe = (stable > num_steps // inner_recurrence)[0].nonzero()
            if len(ripe) > 0:
                k = int(ripe[-1]) + 1
                freeze_up_to(k)
            else:
                freeze_nothing()
                k = 0
        elif freeze_strategy == "fixed":
            if step > num_steps // inner_recurrence:
                n_clear = states.shape[1] - headway - headway_now
                cache.clear_last_k_entries(n_clear)
                clears += n_clear
                states = states[:, headway_now:, :]
                frozen = torch.cat([frozen, new_tokens[:, :headway_now]], dim=-1)
                if streamer:
                    streamer.put(new_tokens[:, :headway_now].cpu())
            else:
                freeze_nothing()
        else:
            raise ValueError(f"Invalid freeze strategy {freeze_strategy}")

        if step > num_steps:
            seen = frozen[0, old_k:k].tolist() if latent else frozen[0, -headway:].tolist()
            token_stop = bool(stops) and any(t in stops for t in seen)
            crit_stop = bool(model_kwargs["stopping_criteria"](frozen, None)) if "stopping_criteria" in model_kwargs else False
            if token_stop or crit_stop:
                break
        if step > max_diffusion_steps:
            break
        if accel:
            prev_prev_states, old_old_ci = prev_states.clone(), old_ci
        if latent:
            prev_states = states.clone()
        old_ci = ci
        step += 1
        old_k = k

    if streamer:
        streamer.end()
    if getattr(gc, "return_dict_in_generate", False):
        scores = {
            "num_core_forward_passes": passes, "num_tokens_forward": tokens_forward, "num_cache_clears": clears,
            "num_standing_waves": standing, "diffusion_steps": step, "gen_seq_length": current.shape[1], "len_prefill": n_prompt,
            "recurrence_per_position": rec_count[:, :frozen.shape[1]].clone(),
            "token_stable_per_position": stable[:, :frozen.shape[1]].clone(),
        }
        return GenerateOutput(sequences=frozen, past_key_values=cache, scores=scores)
    return frozen
