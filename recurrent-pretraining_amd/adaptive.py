"""Per-token adaptive compute: the per-iteration exit evaluators of the reference
(recpre/raven_modeling_minimal.py:2099-2307, same class names, constructor arguments, thresholds and
`init` / `check` protocol) and its generate_with_adaptive_compute loop (RMM:1552-1749).

The statistics over the vocabulary (entropy, KL divergence, min-p filtered KL) and over the latent
state (relative change, cosine distance) are computed by HIP kernels (csrc/exit_stats.hip); only the
comparison with the threshold and the bookkeeping of who has exited happen on the host, as they do in
the reference.  `reduce=True` (the generate loop's setting): statistics of the last position for the logit
criteria, the mean over positions for the latent criteria; `reduce=False`: one value per position, every
position's logits going through the same kernels, with the reference's broadcasting of the initial state
(a [B] or [B, V] start against [B, S] / [B, S, V] statistics: one sequence, or as many positions as sequences).
"""

from __future__ import annotations

from typing import Callable, Optional, Union

import torch

from . import hip


class PerIterationExitEvaluator:
    """Base class (RMM:2105-2114): check() returns (should_exit [B] bool, outputs or None, exit_values [B])."""

    def init(self, initial_latents: torch.Tensor):
        pass

    def check(self, model, latents: torch.Tensor, aux_inputs: dict):
        raise NotImplementedError()


class NoOpExitEvaluator(PerIterationExitEvaluator):
    """Never exits early (RMM:2117-2125)."""

    def check(self, model, latents, aux_inputs):
        B = latents.shape[0]
        return (torch.zeros(B, device=latents.device, dtype=torch.bool), None, torch.zeros(B, device=latents.device))


class _LogitEvaluator(PerIterationExitEvaluator):
    reduce = True

    def _rows(self, model, latents, aux_inputs):
        """(outputs, logits as rows [R, V], shape the per-row statistics take): the last position's logits, [B], under
        `reduce`; every position's, [B, S], otherwise."""
        outputs = model.predict_from_latents(latents, **aux_inputs)
        logits = outputs.logits
        if self.reduce:
            return outputs, logits[:, -1, :].contiguous(), logits.shape[:1]
        return outputs, logits.reshape(-1, logits.shape[-1]).contiguous(), logits.shape[:2]


class EntropyDiffExitEvaluator(_LogitEvaluator):
    """Exit when the entropy of the next-token distribution stops changing (RMM:2128-2148)."""

    def __init__(self, exit_threshold: Union[str, float] = "auto", reduce: bool = True):
        self.exit_threshold = 1e-3 if exit_threshold == "auto" else float(exit_threshold)
        self.reduce = reduce

    def init(self, initial_latents):
        self.prev_entropy = torch.ones(initial_latents.shape[0], device=initial_latents.device) * 100.0

    def check(self, model, latents, aux_inputs):
        outputs, rows, shape = self._rows(model, latents, aux_inputs)
        entropy = hip.exit_logit_stats(rows, hip.EXIT_ENTROPY).view(*shape)
        exit_values = (entropy - self.prev_entropy).abs()
        self.prev_entropy = entropy
        return exit_values < self.exit_threshold, outputs, exit_values


class KLExitEvaluator(_LogitEvaluator):
    """Exit on a small KL divergence between successive next-token distributions (RMM:2170-2187)."""

    _kind = hip.EXIT_KL

    def __init__(self, model, exit_threshold: Union[str, float] = "auto", reduce: bool = True):
        self.exit_threshold = self._auto if exit_threshold == "auto" else float(exit_threshold)
        self.V = model.config.padded_vocab_size
        self.reduce = reduce

    _auto = 0.001

    def init(self, initial_latents):
        B = initial_latents.shape[0]
        self.prev_log_probs = ((1 / self.V) * torch.ones(B, self.V, device=initial_latents.device)).log()

    def check(self, model, latents, aux_inputs):
        outputs, rows, shape = self._rows(model, latents, aux_inputs)
        if self.prev_log_probs.shape != rows.shape:  # per position: the [B, V] start against [B, S, V], as torch broadcasts it
            self.prev_log_probs = torch.broadcast_to(self.prev_log_probs, (*shape, rows.shape[-1])).reshape(rows.shape).contiguous()
        exit_values = hip.exit_logit_stats(rows, self._kind, self.prev_log_probs).view(*shape)  # also stores the new log-probabilities
        return exit_values < self.exit_threshold, outputs, exit_values


class MinKLExitEvaluator(KLExitEvaluator):
    """The same on min-p filtered distributions (RMM:2190-2216)."""

    _kind = hip.EXIT_MINP_KL
    _auto = 1e-5


class ArgmaxStabilityExitEvaluator(_LogitEvaluator):
    """Exit once the arg-max token has not changed for a number of checks (RMM:2219-2241)."""

    def __init__(self, exit_threshold: Union[str, int] = "auto", reduce: bool = True):
        self.exit_threshold = 5 if exit_threshold == "auto" else int(exit_threshold)
        self.reduce = reduce

    def init(self, initial_latents):
        B, dev = initial_latents.shape[0], initial_latents.device
        self.prev_argmax = torch.ones(B, dtype=torch.long, device=dev) * -1
        self.stable_for_n_steps = torch.zeros(B, dtype=torch.long, device=dev)

    def check(self, model, latents, aux_inputs):
        outputs, rows, shape = self._rows(model, latents, aux_inputs)
        current = hip.argmax(rows).view(*shape)
        self.stable_for_n_steps = torch.where(current == self.prev_argmax, self.stable_for_n_steps + 1,
                                              torch.zeros_like(self.stable_for_n_steps))
        self.prev_argmax = current
        return self.stable_for_n_steps >= self.exit_threshold, outputs, self.stable_for_n_steps


class _LatentEvaluator(PerIterationExitEvaluator):
    def init(self, initial_latents):
        self.prev_latents = initial_latents.clone().detach()

    def _stats(self, latents, want_cos: bool):
        B, S, h = latents.shape
        rel, cos = hip.exit_latent_stats(latents.reshape(B * S, h).contiguous(), self.prev_latents.reshape(B * S, h).contiguous(),
                                         want_rel=not want_cos, want_cos=want_cos)
        self.prev_latents = latents.clone().detach()
        return (cos if want_cos else rel).view(B, S)


class LatentDiffExitEvaluator(_LatentEvaluator):
    """Exit on a small relative change of the latent state (RMM:2151-2167)."""

    def __init__(self, exit_threshold: Union[str, float] = "auto", reduce: bool = True):
        self.exit_threshold = 0.03 if exit_threshold == "auto" else float(exit_threshold)
        self.reduce = reduce

    def check(self, model, latents, aux_inputs):
        exit_values = self._stats(latents, want_cos=False)
        if self.reduce:
            exit_values = exit_values.mean(dim=-1)
        return exit_values < self.exit_threshold, None, exit_values


class CosineExitEvaluator(_LatentEvaluator):
    """Exit when successive latent states point the same way (RMM:2244-2260)."""

    def __init__(self, exit_threshold: Union[str, float] = "auto", reduce: bool = True):
        self.exit_threshold = 1e-3 if exit_threshold == "auto" else float(exit_threshold)
        self.reduce = reduce

    def check(self, model, latents, aux_inputs):
        cosine = self._stats(latents, want_cos=True)
        exit_values = 1 - (cosine.mean(dim=1) if self.reduce else cosine)
        return exit_values < self.exit_threshold, None, exit_values


class NumStepsGenerator(PerIterationExitEvaluator):
    """Exits every token after steps_fn(token index) recurrences (RMM:2262-2281)."""

    def __init__(self, steps_fn: Callable):
        self.steps_fn = steps_fn
        self.counter = 0
        self.target_steps = 0
        self.current_step = 0

    def init(self, initial_latents):
        self.target_steps = self.steps_fn(self.counter)
        self.counter += 1
        self.current_step = 0

    def check(self, model, latents, aux_inputs):
        self.current_step += 1
        B, dev = latents.shape[0], latents.device
        return (torch.full((B,), self.current_step >= self.target_steps, dtype=torch.bool, device=dev), None,
                torch.zeros(B, device=dev))


def get_adaptive_exit_evaluator(model, criterion: str, exit_threshold: Union[str, float, int], reduce: bool = True):
    """Factory of RMM:2284-2307."""
    if criterion == "entropy-diff":
        return EntropyDiffExitEvaluator(exit_threshold, reduce)
    if criterion == "latent-diff":
        return LatentDiffExitEvaluator(exit_threshold, reduce)
    if criterion == "cosine":
        return CosineExitEvaluator(exit_threshold, reduce)
    if "kl" in criterion:
        return MinKLExitEvaluator(model, exit_threshold, reduce) if criterion == "minp-kl" else KLExitEvaluator(model, exit_threshold, reduce)
    if criterion == "argmax-stability":
        return ArgmaxStabilityExitEvaluator(exit_threshold, reduce)
    if criterion == "none":
        return NoOpExitEvaluator()
    raise ValueError(f"Invalid adaptive compute strategy: {criterion}")


@torch.no_grad()
def generate_with_adaptive_compute(model, input_ids: torch.Tensor, generation_config=None, tokenizer=None, streamer=None,
                                   continuous_compute: bool = False, criterion: str = "none",
                                   exit_threshold: Union[str, float, int] = "auto", init_scale: float = 1.0,
                                   cache_lookup_strategy: str = "full", do_not_exit_in_prefill: bool = False, min_steps: int = 0,
                                   check_criterion_every_n_steps: int = 1,
                                   exit_evaluator: Optional[PerIterationExitEvaluator] = None,
                                   input_states_fn: Optional[Callable] = None, stop_tokens: Optional[set] = None, **model_kwargs):
    """RMM:1552-1749.  Per token: embed (prelude), then recurrences one at a time through iterate_one_step, asking
    the exit evaluator after each; a sequence's next-token logits are frozen at the step where it met the criterion
    while the batch keeps iterating until every sequence has (or max_steps).  Tokens that stop early leave their
    deeper cache steps empty; later tokens that go deeper resolve them through the cache's lookup strategy, inside
    the attention kernels.  The recurrences are launched eagerly: replaying them from captured HIP graphs (one per
    recurrence index) was built and measured and gained nothing at the 3.5b shape -- the host reads the exit decision
    after every recurrence, and the GPU is not waiting for launches in between.

    Extensions: input_states_fn(token_step, (B, S, h)) supplies the initial latent state of each token step
    (the reference draws it from the device RNG); stop_tokens overrides the reference's fixed stop set; with
    return_dict_in_generate the output's `scores` carries "compute_steps" and "exit_values" per token and sequence
    (the reference builds both and then drops them)."""
    from .modeling import GenerateOutput

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
    max_steps = model_kwargs.get("num_steps", model.config.mean_recurrence)
    stops = model._get_stops(gc) if stop_tokens is None else set(stop_tokens)
    dev = model.device
    input_ids = input_ids.to(dev)
    total = min(prompt_len + max_new, model.config.block_size)
    cache = model._generation_cache(model_kwargs, cache_lookup_strategy, input_ids.shape[0], total)
    h = model.config.n_embd

    def draw(token_step: int, shape, embeds):
        if input_states_fn is not None:
            return input_states_fn(token_step, shape).to(dev, model.dtype)
        return model.initialize_state(embeds, scale=init_scale)

    next_states = None
    if continuous_compute:  # RMM:1589-1591: the first state covers the whole prompt
        embeds0 = None if input_states_fn is not None else model.embed_inputs(input_ids)[0]
        next_states = draw(0, (B, prompt_len, h), embeds0)
    unfinished = [True] * B
    if exit_evaluator is None:
        exit_evaluator = get_adaptive_exit_evaluator(model, criterion, exit_threshold)
    compute_steps = []

    for token_step in range(max_new):
        seen = cache.get_seq_length()
        pos = torch.arange(seen, input_ids.shape[1], device=dev)
        aux_inputs = {"cache_position": pos, "past_key_values": cache, "attention_mask": None}
        embedded, block_idx = model.embed_inputs(input_ids[:, seen:].contiguous(), **aux_inputs)
        current = next_states if continuous_compute else draw(token_step, tuple(embedded.shape), embedded)
        if continuous_compute:
            next_states = current[:, -1:, :].clone()
        exit_values_per_seq = [[] for _ in range(B)]
        compute_steps_per_seq = [0] * B
        # who has left / finished is kept on the host: one device-to-host read per check (its exit flags and values)
        exit_reached = [False] * B
        outputs, next_token_logits = None, None
        exit_evaluator.init(current)
        finished_loop = True

        def rows(flags):
            return torch.tensor(flags, dtype=torch.bool, device=dev)

        for compute_step in range(max_steps):
            current, block_idx, _ = model.iterate_one_step(embedded, current, block_idx=block_idx, **aux_inputs,
                                                           current_step=compute_step)
            if (compute_step < min_steps or (compute_step - min_steps) % check_criterion_every_n_steps != 0
                    or (do_not_exit_in_prefill and token_step == 0)):
                continue
            new_exits, outputs, exit_values = exit_evaluator.check(model, current, aux_inputs)
            host = torch.stack([new_exits.to(torch.float64), exit_values.to(torch.float64)]).tolist()
            running = [not exit_reached[i] and unfinished[i] for i in range(B)]
            for i in range(B):
                if running[i]:
                    exit_values_per_seq[i].append(host[1][i])
            leaving = [bool(host[0][i]) and running[i] for i in range(B)]
            if any(leaving):
                exit_reached = [exit_reached[i] or leaving[i] for i in range(B)]
                if outputs is None:  # latent criteria: the coda and the head run only when somebody leaves
                    outputs = model.predict_from_latents(current, **aux_inputs)
                logits = outputs.logits
                if next_token_logits is None:
                    next_token_logits = logits[:, -1, :].to(torch.float32).clone()
                elif all(leaving):
                    next_token_logits.copy_(logits[:, -1, :])
                else:
                    mask = rows(leaving)
                    next_token_logits[mask] = logits[mask, -1, :].to(torch.float32)
                for i in range(B):
                    if leaving[i]:
                        compute_steps_per_seq[i] = compute_step + 1
                if continuous_compute:
                    mask = rows(leaving)
                    next_states[mask] = current[mask, -1:, :]
            if all(exit_reached[i] or not unfinished[i] for i in range(B)):
                finished_loop = False
                break
        if finished_loop:  # nobody ended the loop early: the remaining sequences take the last outputs
            if outputs is None:
                outputs = model.predict_from_latents(current, **aux_inputs)
            if next_token_logits is None:
                next_token_logits = outputs.logits[:, -1, :].to(torch.float32).clone()
                compute_steps_per_seq = [max_steps] * B
            else:
                for i in range(B):
                    if not exit_reached[i] and unfinished[i]:
                        next_token_logits[i] = outputs.logits[i, -1, :].to(torch.float32)
                        compute_steps_per_seq[i] = max_steps
        if continuous_compute:
            still_running = rows([not exit_reached[i] and unfinished[i] for i in range(B)])
            next_states[still_running] = current[still_running, -1:, :]
        compute_steps.append([compute_steps_per_seq, exit_values_per_seq])

        next_token = model._sample_next_token(next_token_logits, input_ids, gc)
        input_ids = torch.cat([input_ids, next_token], dim=-1)
        if streamer:
            streamer.put(next_token.cpu())
        if stops:
            for i, v in enumerate(next_token.view(-1).tolist()):
                if v in stops:
                    unfinished[i] = False
        if "stopping_criteria" in model_kwargs:
            done = model_kwargs["stopping_criteria"](input_ids, None).tolist()
            unfinished = [unfinished[i] and not done[i] for i in range(B)]
        if not any(unfinished):
            break
    if streamer:
        streamer.end()
    if getattr(gc, "return_dict_in_generate", False):
        steps_taken, exit_values = zip(*compute_steps)
        return GenerateOutput(sequences=input_ids, past_key_values=cache,
                              scores={"compute_steps": list(steps_taken), "exit_values": list(exit_values)})
    return input_ids


@torch.no_grad()
def prefill_with_varied_exit_steps(model, input_ids: torch.Tensor, exit_evaluator: PerIterationExitEvaluator,
                                   past_key_values=None, init_scale: float = 1.0, input_states_fn: Optional[Callable] = None,
                                   **kwargs):
    """RMM:937-996: the opposite of a real prefill -- token by token, each token leaves the recurrence as soon as
    the evaluator says so.  Returns (logits [1, S, V] float, cache, compute steps per token)."""
    from .cache import HuginnDynamicCache

    assert input_ids.shape[0] == 1  # the reference's restriction (RMM:950)
    cache = past_key_values if past_key_values is not None else HuginnDynamicCache()
    dev = model.device
    input_ids = input_ids.to(dev)
    rows, compute_steps = [], []
    for p in range(input_ids.shape[1]):
        aux_inputs = {"cache_position": torch.tensor([p], device=dev), "past_key_values": cache, "attention_mask": None}
        embedded, block_idx = model.embed_inputs(input_ids[:, p:p + 1].contiguous(), **aux_inputs)
        if input_states_fn is not None:
            current = input_states_fn(p, tuple(embedded.shape)).to(dev, model.dtype)
        else:
            current = model.initialize_state(embedded, scale=init_scale)
        exit_evaluator.init(current)
        compute_step = -1
        for compute_step in range(model.config.mean_recurrence):
            current, block_idx, _ = model.iterate_one_step(embedded, current, block_idx=block_idx, **aux_inputs,
                                                           current_step=compute_step)
            new_exits, _, _ = exit_evaluator.check(model, current, aux_inputs)
            if bool(new_exits.any()):
                break
        compute_steps.append(compute_step + 1)
        rows.append(model.predict_from_latents(current, **aux_inputs).logits)
    return torch.cat(rows, dim=1), cache, compute_steps


@torch.no_grad()
def forward_with_adaptive_compute(model, input_ids: torch.Tensor, exit_evaluator: PerIterationExitEvaluator, labels=None,
                                  past_key_values=None, output_details: Optional[dict] = None, init_scale: float = 1.0,
                                  **kwargs):
    """RMM:998-1035: token-by-token forward with per-token exits; `stats["compute_steps"]` lists the steps taken."""
    from .modeling import CausalLMOutputRecurrentLatents

    logits, _, compute_steps = prefill_with_varied_exit_steps(model, input_ids, exit_evaluator, past_key_values, init_scale, **kwargs)
    if labels is not None:
        loss = torch.nn.functional.cross_entropy(logits.view(-1, logits.shape[-1]), labels.to(logits.device).view(-1))
        log_ppl = loss.clone().detach()
    else:
        loss, log_ppl = torch.as_tensor(0.0), torch.as_tensor(0.0)
    keep = output_details is None or output_details.get("return_logits", True)
    return CausalLMOutputRecurrentLatents(loss=loss, log_ppl=log_ppl, logits=logits if keep else None,
                                          stats={"compute_steps": compute_steps})
