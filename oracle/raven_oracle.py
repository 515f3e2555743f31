"""CPU oracle for the Huginn/Raven recurrent-core decode path.  TEST INFRASTRUCTURE ONLY.

This file restates, with plain PyTorch CPU ops, the arithmetic of the reference's
inference model (recpre/raven_modeling_minimal.py, "RMM" below).  It is the checker the
HIP kernels are compared with; nothing in the shipped package may import it.  Only
tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py use it.

Every function names the reference lines it follows.  Rounding points are the ones a
dtype-cast reference model has (no autocast): each nn.Linear output, each elementwise
result and each norm output is stored in the model dtype; reductions, softmax and
RoPE run in fp32.

How each function is pinned (tests/test_oracle_pins.py), without running the reference:
  rmsnorm            closed forms (constant rows, one-hot rows), F.rms_norm cross-check,
                     fp64 brute force, rounding-order test                       -> pinned
  rope_table/apply   complex multiplication form, pos=0 identity, norm preservation,
                     relative-position property, spot values                     -> pinned
  DictCache          brute-force list model, step enumeration, seen-token law,
                     cache-size known answers from the reference notebooks       -> pinned
  attention          eager softmax(QK^T/sqrt d)V in fp64, T=1 and q=0 special cases,
                     torch SDPA library cross-check                               -> pinned
  linear/adapter     fp64 matmul, split-concat identity, swapped-order negative   -> pinned
  gated_mlp          fp64 restatement, gate-half negative test                    -> pinned
  block/iterate/forward/greedy   composition laws (r=0, cache vs no-cache,
                     prefill-then-decode vs token-by-token)                       -> pinned
  initialize_state   bounds, std, scale=0, generator determinism                  -> pinned
  DictCache lookups  (latest-m4, available-m4, always-last-m4, skip, randomized) closed form on
                     step-tagged entries                                          -> pinned
  ExitCriterion      entropy of uniform / one-hot rows, KL(p, p) = 0 and two-point closed
                     form, fp64 brute force, min-p floor by hand, latent ratios of scaled /
                     orthogonal vectors, argmax streak counting                    -> pinned
  embed_inputs / iterate_one_step / predict_from_latents / generate_with_adaptive_compute
                     pieces compose to forward(); criterion "none" equals greedy_generate;
                     num-steps evaluator equals forward(num_steps=k) token by token -> pinned
  generate_diffusion_style   every position of the wave recomputed one position at a time, without a step-indexed
                     cache, roll-back or batching (each position keeps the key/value rows of its own last
                     computation; tokens, embedding averages, noise damping and the freeze rule restated per
                     position): states and logits of all wave positions after every step and the frozen text, for
                     "fixed" and for "latent-diff" at two thresholds with waves up to 12 wide; the leftmost
                     position also by hand on a copy of the prompt cache; schedule / counter closed forms for
                     "fixed" and for exit thresholds 0 and infinity                  -> pinned
  inject_noise       amplitude n = t * sqrt(2/5) and the per-type coefficients (n/(k+1), n/sqrt(k+1), max(n, (r-k)/r),
                     2un) by closed form on x = 0 / noise = 1; zero noise leaves norm_4(x) (scale invariance);
                     "line" at step 0 replaces the state, so forward() no longer depends on input_states;
                     the roundings against the reference's expression evaluated by torch ON THE GPU
                     (tests/test_gpu_model.py)                                        -> pinned
The reference holds no golden vectors for this path (it has no test suite); the only
exact numbers it publishes are three KV-cache sizes, used as known-answer tests.
"""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional

import torch
import torch.nn.functional as F


# --------------------------------------------------------------------------------------
# shape / config  (recpre/raven_config_minimal.py:12-91)
# --------------------------------------------------------------------------------------
@dataclass
class RavenShape:
    n_embd: int = 5280
    n_heads: int = 55
    intermediate_size: int = 17920
    vocab_size: int = 65536
    n_layers_in_prelude: int = 2
    n_layers_in_recurrent_block: int = 4
    n_layers_in_coda: int = 2
    mean_recurrence: int = 32
    block_size: int = 4096
    rope_base: float = 50000.0
    norm_eps: float = 1e-6
    qk_bias: bool = True
    test_time_noise: float = 0.0
    test_time_noise_type: str = "fixed"

    @property
    def head_dim(self) -> int:
        return self.n_embd // self.n_heads

    @property
    def emb_scale(self) -> float:  # RMM:27-33, 50-52
        return math.sqrt(self.n_embd)

    @property
    def init_std(self) -> float:  # raven_config_minimal.py:86
        return math.sqrt(2.0 / (5.0 * self.n_embd))

    @staticmethod
    def nebel() -> "RavenShape":
        return RavenShape()

    @staticmethod
    def tiny() -> "RavenShape":
        return RavenShape(
            n_embd=256, n_heads=4, intermediate_size=704, vocab_size=1024,
            n_layers_in_prelude=1, n_layers_in_recurrent_block=2, n_layers_in_coda=1,
            mean_recurrence=4,
        )


def block_keys(prefix: str, qk_bias: bool = True) -> list[str]:
    """State-dict names of one SandwichBlock, in module registration order (RMM:515-523, 440-452, 497-503)."""
    keys = [f"{prefix}.norm_1.weight", f"{prefix}.attn.Wqkv.weight"]
    if qk_bias:
        keys.append(f"{prefix}.attn.qk_bias")
    keys += [
        f"{prefix}.attn.proj.weight", f"{prefix}.norm_2.weight",
        f"{prefix}.mlp.fc.weight", f"{prefix}.mlp.proj.weight",
        f"{prefix}.norm_3.weight", f"{prefix}.norm_4.weight",
    ]
    return keys


def state_dict_layout(s: RavenShape) -> list[tuple[str, tuple[int, ...]]]:
    """(name, shape) of every tensor of the interchange format, in registration order (RMM:551-577)."""
    h, hd, nh, inter = s.n_embd, s.head_dim, s.n_heads, s.intermediate_size

    def blk(prefix):
        shapes = {
            "norm_1.weight": (h,), "norm_2.weight": (h,), "norm_3.weight": (h,), "norm_4.weight": (h,),
            "attn.Wqkv.weight": (3 * h, h), "attn.qk_bias": (2, 1, nh, hd), "attn.proj.weight": (h, h),
            "mlp.fc.weight": (2 * inter, h), "mlp.proj.weight": (h, inter),
        }
        return [(k, shapes[k[len(prefix) + 1:]]) for k in block_keys(prefix, s.qk_bias)]

    out = [("transformer.wte.weight", (s.vocab_size, h))]
    for i in range(s.n_layers_in_prelude):
        out += blk(f"transformer.prelude.{i}")
    out.append(("transformer.adapter.weight", (h, 2 * h)))
    for i in range(s.n_layers_in_recurrent_block):
        out += blk(f"transformer.core_block.{i}")
    for i in range(s.n_layers_in_coda):
        out += blk(f"transformer.coda.{i}")
    out.append(("transformer.ln_f.weight", (h,)))
    return out


def make_weights(s: RavenShape, seed: int = 0, dtype=torch.float32, only_core: bool = False) -> dict[str, torch.Tensor]:
    """Seeded synthetic weights: matrices, embedding and qk_bias ~ N(0, 0.02); norm weights ~ N(1, 0.02).

    One CPU generator, one draw per tensor in state-dict order, drawn in fp32 and then cast, so any
    host reproduces the same values.  lm_head is tied to wte (RMM:574-575).  `only_core` restricts the
    draw to the adapter and core blocks (what one recurrence iteration touches); that subset uses its
    own stream and does not equal the same tensors of the full draw.
    """
    g = torch.Generator(device="cpu").manual_seed(seed)
    w: dict[str, torch.Tensor] = {}
    for name, shape in state_dict_layout(s):
        if only_core and not (name.startswith("transformer.core_block") or name.startswith("transformer.adapter")):
            continue
        mean = 1.0 if (name.endswith("weight") and len(shape) == 1) else 0.0
        t = torch.empty(shape, dtype=torch.float32).normal_(mean, 0.02, generator=g)
        w[name] = t.to(dtype)
    if not only_core:
        w["lm_head.weight"] = w["transformer.wte.weight"]
        w["freqs_cis"] = rope_table(s.head_dim, s.block_size, s.rope_base)
    return w


# --------------------------------------------------------------------------------------
# elementary ops
# --------------------------------------------------------------------------------------
LINEAR_MODE = "native"


def set_linear_mode(mode: str) -> None:
    """'native': nn.Linear semantics in the tensor's own dtype, what the reference executes.
    'f32': upcast both operands, multiply in fp32, round once to the input dtype -- the same
    mathematics with another accumulation order; the distance between the two modes is the
    accumulation-order sensitivity that composed bf16 results are judged against."""
    global LINEAR_MODE
    assert mode in ("native", "f32")
    LINEAR_MODE = mode


def linear(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    if LINEAR_MODE == "f32" and x.dtype != torch.float32:
        return F.linear(x.float(), w.float()).to(x.dtype)
    return F.linear(x, w)


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """RMM:137-142.  Normalise in fp32, cast to x's dtype, THEN scale by the weight in that dtype."""
    x32 = x.float()
    inv = torch.rsqrt(x32.pow(2).mean(dim=-1, keepdim=True) + eps)
    return (x32 * inv).to(x.dtype) * weight


def rope_table(head_dim: int, n_pos: int, base: float) -> torch.Tensor:
    """RMM:2076-2081 with condense_ratio 1.  fp32 table [1, n_pos, 1, head_dim/2, 2] of (cos, sin)."""
    expo = torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim
    inv_freq = 1.0 / (base ** expo)
    ang = torch.outer(torch.arange(n_pos, dtype=torch.float32), inv_freq).float()
    return torch.stack([ang.cos()[None, :, None, :], ang.sin()[None, :, None, :]], dim=4)


def apply_rope(q: torch.Tensor, k: torch.Tensor, freqs: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """RMM:2087-2098.  q,k [B,S,nh,hd]; freqs [1,S,1,hd/2,2].  Adjacent element pairs are rotated in fp32."""
    def rot(t):
        p = t.float().unflatten(-1, (-1, 2))
        c, s_ = freqs[..., 0], freqs[..., 1]
        out = torch.stack([p[..., 0] * c - p[..., 1] * s_, p[..., 1] * c + p[..., 0] * s_], dim=-1)
        return out.flatten(3).to(t.dtype)
    return rot(q), rot(k)


def remap_step(step_idx: int, strategy: str) -> int:
    """Cache-sharing remap of the step slot, RMM:169-182 (hard-codes 2 prelude and 4 core blocks)."""
    if "compress-" in strategy and step_idx > 1:
        if "compress-s" in strategy:
            n = int(strategy.split("compress-")[1][1:])
            return (step_idx - 2) % n + 2
        if "compress-anchor" in strategy:
            return step_idx if step_idx - 2 < 32 else 34 + (step_idx - 34) % 4
        n = int(strategy.split("compress-")[1][1:])
        return (step_idx - 2) // n + 2
    return step_idx


class DictCache:
    """Brute-force model of HuginnDynamicCache (RMM:148-308): cache[step][position] -> [B, nh, hd] tensor."""

    def __init__(self, lookup_strategy: str = "full"):
        self._seen_tokens = 0
        self.key_cache: dict[int, dict[int, torch.Tensor]] = {}
        self.value_cache: dict[int, dict[int, torch.Tensor]] = {}
        self.lookup_strategy = lookup_strategy

    def update(self, k: torch.Tensor, v: torch.Tensor, step_idx, lookup_strategy: Optional[str] = None):
        """k, v: [B, nh, S, hd].  Returns the stacked K, V of that step, [B, nh, T, hd] (RMM:160-204)."""
        step = remap_step(int(step_idx), self.lookup_strategy)
        lookup = self.lookup_strategy if lookup_strategy is None else lookup_strategy
        n_new = k.shape[-2]
        kc = self.key_cache.setdefault(step, {})
        vc = self.value_cache.setdefault(step, {})
        if step == 0:                                   # RMM:188-189
            self._seen_tokens += n_new
        first = self._seen_tokens - n_new
        for i in range(n_new):
            if "compress-" not in self.lookup_strategy:  # RMM:192-193
                assert step < 0 or (first + i) not in kc, "overwrite of a cached position"
            kc[first + i] = k[..., i, :]
            vc[first + i] = v[..., i, :]
        if len(kc) == self._seen_tokens or self.lookup_strategy == "full":
            return torch.stack(list(kc.values()), dim=-2), torch.stack(list(vc.values()), dim=-2)
        return self._lookup_partial(step, lookup)

    def _lookup_partial(self, step: int, lookup: str):
        """Fallbacks when some positions were never computed at this step (RMM:206-273)."""
        ks, vs = [], []
        for pos in range(self._seen_tokens):
            if lookup.startswith("latest-m4") or lookup.startswith("always-last-m4"):
                if step >= 2:
                    pool = range(step + 1) if lookup.startswith("latest-m4") else list(self.key_cache)
                    have = [s for s in pool if pos in self.key_cache.get(s, {})]
                    src = max(s for s in have if s >= 2 and s % 4 == step % 4)
                else:
                    src = step if pos in self.key_cache[step] else 0
            elif lookup.startswith("available-m4"):
                if pos in self.key_cache[step]:
                    src = step
                else:
                    have = [s for s in range(step + 1) if pos in self.key_cache.get(s, {})]
                    src = max(s for s in have if s >= 2 and s % 4 == step % 4)
            elif lookup.startswith("skip"):
                if pos not in self.key_cache[step]:
                    continue
                src = step
            elif lookup.startswith("randomized"):       # RMM:255-271: one CPU draw per position, in position order
                if step < 2:
                    src = step if pos in self.key_cache[step] else 0
                else:
                    block = (step - 2) % 4 + 2
                    have = [s for s in range(2, step + 1) if (s - 2) % 4 + 2 == block and pos in self.key_cache[s]]
                    src = have[torch.randint(len(have), (1,))]
            else:
                raise ValueError(f"Unknown lookup strategy: {lookup}")
            ks.append(self.key_cache[src][pos])
            vs.append(self.value_cache[src][pos])
        return torch.stack(ks, dim=-2), torch.stack(vs, dim=-2)

    def reset(self):  # RMM:275-279
        self._seen_tokens = 0
        self.key_cache.clear()
        self.value_cache.clear()

    def clear_last_k_entries(self, k: int = 0):  # RMM:281-293
        assert self._seen_tokens >= k
        self._seen_tokens -= k
        keep = self._seen_tokens
        self.key_cache = {s: {p: t for p, t in c.items() if p < keep} for s, c in self.key_cache.items()}
        self.value_cache = {s: {p: t for p, t in c.items() if p < keep} for s, c in self.value_cache.items()}

    def get_seq_length(self, step_idx: int = 0) -> int:  # RMM:295-296
        return self._seen_tokens

    def get_memory_usage(self) -> float:  # RMM:298-308: key bytes, doubled, in MiB
        n = sum(t.nelement() * t.element_size() for c in self.key_cache.values() for t in c.values())
        return n * 2 / (1024 * 1024)


def sdpa(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    """The three mask cases of RMM:484-491, written out as an explicit fp32 softmax.

    q [B,nh,Sq,hd], k/v [B,nh,Sk,hd].  Sq == Sk: causal.  1 < Sq < Sk: causal aligned to the
    lower-right corner (query i sees keys 0 .. Sk-Sq+i).  Sq == 1: no mask.  Scale 1/sqrt(hd).
    """
    sq, sk = q.shape[-2], k.shape[-2]
    scores = (q.float() @ k.float().transpose(-1, -2)) / math.sqrt(q.shape[-1])
    if sq > 1:
        qi = torch.arange(sq)[:, None]
        kj = torch.arange(sk)[None, :]
        scores = scores.masked_fill(kj > qi + (sk - sq), float("-inf"))
    return (torch.softmax(scores, dim=-1) @ v.float()).to(q.dtype)


def attention(x, w, prefix, freqs, step_idx, cache, s: RavenShape):
    """CausalSelfAttention.forward, RMM:454-493.  x [B,S,h] is the already-normalised input."""
    b, sq, h = x.shape
    nh, hd = s.n_heads, s.head_dim
    qkv = linear(x, w[f"{prefix}.attn.Wqkv.weight"])
    q, k, v = (t.view(b, sq, nh, hd) for t in qkv.split([h, h, h], dim=2))
    if s.qk_bias:
        bias = w[f"{prefix}.attn.qk_bias"]
        q, k = (q + bias[0:1]).to(q.dtype), (k + bias[1:2]).to(q.dtype)
    q, k = apply_rope(q, k, freqs)
    q, k, v = q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2)
    if cache is not None:
        k, v = cache.update(k, v, step_idx)
    y = sdpa(q, k, v)
    y = y.transpose(1, 2).reshape(b, sq, h)
    return linear(y, w[f"{prefix}.attn.proj.weight"])


def gated_mlp(x, w, prefix):
    """GatedMLP.forward, RMM:505-509.  The gate is the FIRST half of fc's output."""
    gate, up = linear(x, w[f"{prefix}.mlp.fc.weight"]).chunk(2, dim=-1)
    return linear(F.silu(gate) * up, w[f"{prefix}.mlp.proj.weight"])


def sandwich_block(x, w, prefix, freqs, step_idx, cache, s: RavenShape):
    """SandwichBlock.forward, RMM:525-536."""
    eps = s.norm_eps
    a = attention(rmsnorm(x, w[f"{prefix}.norm_1.weight"], eps), w, prefix, freqs, step_idx, cache, s)
    x = rmsnorm(a + x, w[f"{prefix}.norm_2.weight"], eps)
    m = gated_mlp(rmsnorm(x, w[f"{prefix}.norm_3.weight"], eps), w, prefix)
    return rmsnorm(m + x, w[f"{prefix}.norm_4.weight"], eps)


def inject_noise(x, current_step: int, w, s: RavenShape, draws=None, renorm: bool = True):
    """RMM:815-837: x <- x * (1 - c) + randn_like(x) * c with c from the noise type and the recurrence index, then the
    last core block's norm_4 again.  `draws` supplies the random numbers (normal(x), uniform(x)) so that a checker and a
    checked run can share them.

    Every product, quotient and sum of the reference's expression is one elementwise torch op and rounds to the state's
    dtype.  Its operands are Python floats (the elementwise GPU kernels take them as float32) and, for "geom" and
    "sqrt", 0-dim float32 tensors ON THE DEVICE: ATen's GPU kernels convert such an operand to the result dtype before
    the operation (torch on the CPU keeps it in float32 -- the two differ, so the roundings are spelled out here
    rather than left to CPU torch's promotion)."""
    if s.test_time_noise <= 0:
        return x
    dt = x.dtype
    f = lambda v: torch.tensor(v, dtype=torch.float32)
    dev0 = lambda v: v.to(dt).float()          # a 0-dim device tensor as the GPU kernel takes it
    rnd = lambda v: v.to(dt).float()           # the rounding of an op's result
    n = s.test_time_noise * s.init_std * s.emb_scale
    kind = s.test_time_noise_type
    if kind == "chi":                          # the reference draws the amplitude before the noise
        u = (draws.uniform(x) if draws is not None else torch.rand(1, dtype=dt)).to(dt).float()
    noise = (draws.normal(x) if draws is not None else torch.randn_like(x)).to(dt).float()
    if kind in ("geom", "sqrt"):               # RMM:818-823
        d = f(current_step + 1) if kind == "geom" else f(current_step + 1).sqrt()
        keep = dev0(1 - f(n) / d)
        mixed = rnd(rnd(noise * f(n)) / dev0(d))
    elif kind == "line":                       # RMM:824-826
        c = max(n, (s.mean_recurrence - current_step) / s.mean_recurrence)
        keep, mixed = f(1 - c), rnd(noise * f(c))
    elif kind == "chi":                        # RMM:827-829
        c = rnd(rnd(2 * u) * f(n))
        keep, mixed = rnd(1 - c), rnd(noise * c)
    elif kind == "fixed":                      # RMM:830-831
        keep, mixed = f(1 - n), rnd(noise * f(n))
    else:
        raise ValueError(kind)
    x = (rnd(x.float() * keep) + mixed).to(dt)
    if renorm:
        last = s.n_layers_in_recurrent_block - 1
        x = rmsnorm(x, w[f"transformer.core_block.{last}.norm_4.weight"], s.norm_eps)
    return x


def core_block_forward(x, embeds, w, freqs, cache, block_idx: int, s: RavenShape, current_step: int = 0, noise_draws=None):
    """RMM:764-781.  Adapter input order is (state, embedded input)."""
    x = inject_noise(x, current_step, w, s, noise_draws)
    x = linear(torch.cat([x, embeds], dim=-1), w["transformer.adapter.weight"])
    for j in range(s.n_layers_in_recurrent_block):
        block_idx += 1
        x = sandwich_block(x, w, f"transformer.core_block.{j}", freqs, block_idx, cache, s)
    return x, block_idx


def initialize_state(embeds: torch.Tensor, s: RavenShape, scale: float = 1.0,
                     generator: Optional[torch.Generator] = None) -> torch.Tensor:
    """RMM:804-813.  randn draw (discarded), truncated normal +-3 std, then times sqrt(n_embd)."""
    x = torch.empty_like(embeds).normal_(generator=generator)
    std = s.init_std * scale
    if std > 0:
        torch.nn.init.trunc_normal_(x, mean=0.0, std=std, a=-3 * std, b=3 * std, generator=generator)
        x = x * s.emb_scale
    else:
        x.zero_()
    return x


def split_num_steps(num_steps, s: RavenShape) -> tuple[int, int]:
    """RMM:739-744 and the eval branch of the sampler, RMM:799-802."""
    if num_steps is None:
        return s.mean_recurrence, 0
    if isinstance(num_steps, torch.Tensor) and num_steps.dim() == 0:  # a 0-d tensor counts as an int
        return int(num_steps), 0
    if hasattr(num_steps, "__len__") and len(num_steps) > 1:
        return int(num_steps[0]), int(num_steps[1])
    return int(num_steps), 0


def iterate_forward(embeds, input_states, w, freqs, block_idx: int, cache, num_steps, s: RavenShape,
                    init_scale: float = 1.0, generator=None, noise_draws=None):
    """RMM:726-762 (inference: the no-grad and grad loops do the same arithmetic and number their steps through)."""
    x = initialize_state(embeds, s, init_scale, generator) if input_states is None else input_states.clone()
    n0, n1 = split_num_steps(num_steps, s)
    for step in range(n0 + n1):
        x, block_idx = core_block_forward(x, embeds, w, freqs, cache, block_idx, s, step, noise_draws)
    return rmsnorm(x, w["transformer.ln_f.weight"], s.norm_eps), block_idx


def pick_freqs(table: torch.Tensor, n_tokens: int, position_ids=None, cache_position=None):
    """Position selection shared by forward / iterate_one_step / predict_from_latents (RMM:660-665)."""
    if position_ids is None and cache_position is None:
        return table[:, :n_tokens]
    if position_ids is not None:
        return table.index_select(1, position_ids.squeeze())
    return table[:, cache_position]


@dataclass
class OracleOutput:
    logits: torch.Tensor
    latent_states: torch.Tensor
    past_key_values: Optional[DictCache] = None
    hidden_states: Optional[torch.Tensor] = None


def forward(w, s: RavenShape, input_ids=None, input_embeds=None, input_states=None, position_ids=None,
            num_steps=None, past_key_values=None, use_cache=False, cache_position=None, init_scale=1.0,
            generator=None, noise_draws=None) -> OracleOutput:
    """RavenForCausalLM.forward, RMM:638-724 (labels / stats branches left out; attention_mask is ignored there)."""
    n_tok = input_ids.shape[1] if input_ids is not None else input_embeds.shape[1]
    freqs = pick_freqs(w["freqs_cis"], n_tok, position_ids, cache_position)
    if input_embeds is None:
        input_embeds = F.embedding(input_ids, w["transformer.wte.weight"])
    input_embeds = input_embeds * s.emb_scale
    if use_cache and past_key_values is None:
        past_key_values = DictCache()
    cache = past_key_values
    block_idx = -1
    for i in range(s.n_layers_in_prelude):
        block_idx += 1
        input_embeds = sandwich_block(input_embeds, w, f"transformer.prelude.{i}", freqs, block_idx, cache, s)
    x, block_idx = iterate_forward(input_embeds, input_states, w, freqs, block_idx, cache, num_steps, s,
                                   init_scale, generator, noise_draws)
    latents = x.clone()
    block_idx = 0
    for i in range(s.n_layers_in_coda):
        block_idx -= 1
        x = sandwich_block(x, w, f"transformer.coda.{i}", freqs, block_idx, cache, s)
    x = rmsnorm(x, w["transformer.ln_f.weight"], s.norm_eps)
    logits = linear(x, w["lm_head.weight"]).float()
    return OracleOutput(logits=logits, latent_states=latents, past_key_values=cache, hidden_states=x)


def repetition_penalty(logits: torch.Tensor, ids: torch.Tensor, penalty: float) -> torch.Tensor:
    """The standard penalty of RMM:2047-2061 on [B, V] logits: every token that occurs in the row's sequence so far has
    its logit divided by the penalty when positive and multiplied when negative."""
    out = logits.to(copy=True, dtype=torch.float32)
    for b in range(out.shape[0]):
        seen = torch.unique(ids[b])
        vals = out[b, seen]
        out[b, seen] = torch.where(vals < 0, vals * penalty, vals / penalty)
    return out


def greedy_generate(w, s: RavenShape, input_ids: torch.Tensor, max_new_tokens: int, num_steps=None,
                    state_fn=None, stop_tokens=(), record: Optional[dict] = None,
                    penalty: Optional[float] = None) -> torch.Tensor:
    """The greedy branch of generate_minimal (RMM:1165-1232, argmax at RMM:1988-1989).

    `state_fn(call_index, embeds_shape)` supplies the latent state injected into each forward (the
    reference draws it from the global RNG on every call, RMM:738; parity runs inject it instead).
    `record`, if given, receives per-token top-2 logit margins and the cache object.
    `penalty`: generation_config.repetition_penalty (RMM:1946-1947, 2047-2061).
    """
    cache = DictCache()
    ids = input_ids.clone()
    alive = torch.ones(ids.shape[0], dtype=torch.bool)
    margins = []
    for call in range(max_new_tokens):
        seen = cache.get_seq_length()
        pos = torch.arange(seen, ids.shape[1])
        step_ids = ids[:, pos]
        states = None if state_fn is None else state_fn(call, (ids.shape[0], step_ids.shape[1], s.n_embd))
        out = forward(w, s, input_ids=step_ids, input_states=states, num_steps=num_steps,
                      past_key_values=cache, use_cache=True, cache_position=pos,
                      init_scale=0.0 if state_fn is None else 1.0)
        last = out.logits[:, -1, :].float()
        if penalty is not None and penalty != 1.0:  # RMM:1946-1947: over the whole sequence so far, on every step
            last = repetition_penalty(last, ids, penalty)
        top2 = last.topk(2, dim=-1).values
        margins.append((top2[:, 0] - top2[:, 1]).tolist())
        nxt = last.argmax(dim=-1, keepdim=True)
        ids = torch.cat([ids, nxt], dim=-1)
        for b in range(ids.shape[0]):
            if alive[b] and int(nxt[b, 0]) in stop_tokens:
                alive[b] = False
        if not alive.any():
            break
    if record is not None:
        record["margins"] = margins
        record["cache"] = cache
    return ids


# --------------------------------------------------------------------------------------
# adaptive compute: per-iteration exit criteria and the generate loop around them
# (RMM:841-934 pieces of the forward, 1552-1749 the loop, 2099-2307 the criteria)
# --------------------------------------------------------------------------------------
def embed_inputs(w, s: RavenShape, input_ids, cache=None, cache_position=None, position_ids=None):
    """RMM:902-934: embedding times sqrt(h), then the prelude; returns (embeds, block_idx)."""
    freqs = pick_freqs(w["freqs_cis"], input_ids.shape[1], position_ids, cache_position)
    x = F.embedding(input_ids, w["transformer.wte.weight"]) * s.emb_scale
    block_idx = -1
    for i in range(s.n_layers_in_prelude):
        block_idx += 1
        x = sandwich_block(x, w, f"transformer.prelude.{i}", freqs, block_idx, cache, s)
    return x, block_idx


def iterate_one_step(w, s: RavenShape, embeds, states, block_idx: int, cache=None, cache_position=None, position_ids=None,
                     current_step: int = 0, noise_draws=None):
    """RMM:841-868: one recurrence; returns (state, block_idx)."""
    freqs = pick_freqs(w["freqs_cis"], embeds.shape[1], position_ids, cache_position)
    return core_block_forward(states, embeds, w, freqs, cache, block_idx, s, current_step, noise_draws)


def predict_from_latents(w, s: RavenShape, latents, cache=None, cache_position=None, position_ids=None) -> OracleOutput:
    """RMM:870-900: ln_f, coda (step indices -1, -2, ...), ln_f, tied head, float logits."""
    freqs = pick_freqs(w["freqs_cis"], latents.shape[1], position_ids, cache_position)
    x = rmsnorm(latents, w["transformer.ln_f.weight"], s.norm_eps)
    block_idx = 0
    for i in range(s.n_layers_in_coda):
        block_idx -= 1
        x = sandwich_block(x, w, f"transformer.coda.{i}", freqs, block_idx, cache, s)
    x = rmsnorm(x, w["transformer.ln_f.weight"], s.norm_eps)
    return OracleOutput(logits=linear(x, w["lm_head.weight"]).float(), latent_states=x, past_key_values=cache)


EXIT_AUTO = {"entropy-diff": 1e-3, "latent-diff": 0.03, "cosine": 1e-3, "kl": 1e-3, "minp-kl": 1e-5, "argmax-stability": 5}


class ExitCriterion:
    """The per-iteration exit evaluators of RMM:2099-2307 behind one class (reduce=True, the generate loop's use).

    check(latents, predict) -> (exit?[B] bool, outputs or None, value[B]); `predict` maps latents to an
    OracleOutput (the coda and the head) and is only called by the criteria that look at logits."""

    def __init__(self, criterion: str, threshold="auto", vocab: int = 0, steps_fn=None):
        if criterion == "none" or criterion == "num-steps":
            self.kind = criterion
        elif criterion in ("entropy-diff", "latent-diff", "cosine", "argmax-stability"):
            self.kind = criterion
        elif "kl" in criterion:                      # RMM:2295-2299: any other name containing "kl" is the plain KL
            self.kind = "minp-kl" if criterion == "minp-kl" else "kl"
        else:
            raise ValueError(f"Invalid adaptive compute strategy: {criterion}")
        if self.kind in EXIT_AUTO:
            t = EXIT_AUTO[self.kind] if threshold == "auto" else threshold
            self.threshold = int(t) if self.kind == "argmax-stability" else float(t)
        self.V, self.steps_fn, self.counter = vocab, steps_fn, 0

    def init(self, latents: torch.Tensor) -> None:
        B = latents.shape[0]
        if self.kind == "entropy-diff":
            self.prev = torch.ones(B) * 100.0                                    # RMM:2135-2137
        elif self.kind in ("latent-diff", "cosine"):
            self.prev = latents.clone()                                          # RMM:2156-2157, 2250-2251
        elif self.kind in ("kl", "minp-kl"):
            self.prev = ((1 / self.V) * torch.ones(B, self.V)).log()             # RMM:2175-2177
        elif self.kind == "argmax-stability":
            self.prev = torch.ones(B, dtype=torch.long) * -1                     # RMM:2225-2228
            self.stable = torch.zeros(B, dtype=torch.long)
        elif self.kind == "num-steps":                                           # RMM:2269-2272
            self.target, self.current = self.steps_fn(self.counter), 0
            self.counter += 1

    def check(self, latents: torch.Tensor, predict):
        B = latents.shape[0]
        if self.kind == "none":                                                  # RMM:2120-2125
            return torch.zeros(B, dtype=torch.bool), None, torch.zeros(B)
        if self.kind == "num-steps":                                             # RMM:2274-2281
            self.current += 1
            return torch.full((B,), self.current >= self.target, dtype=torch.bool), None, torch.zeros(B)
        if self.kind == "latent-diff":                                           # RMM:2159-2167
            v = ((latents - self.prev).norm(dim=-1) / latents.norm(dim=-1)).mean(dim=-1)
            self.prev = latents.clone()
            return v < self.threshold, None, v
        if self.kind == "cosine":                                                # RMM:2253-2260
            cos = (latents * self.prev).sum(dim=-1) / latents.norm(dim=-1) / self.prev.norm(dim=-1)
            v = 1 - cos.mean(dim=1)
            self.prev = latents.clone()
            return v < self.threshold, None, v
        out = predict(latents)
        last = out.logits[:, -1, :]
        if self.kind == "entropy-diff":                                          # RMM:2139-2148
            probs = F.softmax(last, dim=-1)
            entropy = -torch.sum(probs * torch.log(probs + 1e-10), dim=-1)
            v = (entropy - self.prev).abs()
            self.prev = entropy
            return v < self.threshold, out, v
        if self.kind == "argmax-stability":                                      # RMM:2230-2241
            cur = last.argmax(dim=-1)
            self.stable = torch.where(cur == self.prev, self.stable + 1, torch.zeros_like(self.stable))
            self.prev = cur
            return self.stable >= self.threshold, out, self.stable
        if self.kind == "kl":                                                    # RMM:2179-2187
            logp = F.log_softmax(last, dim=-1)
        else:                                                                    # RMM:2200-2216
            probs = F.softmax(last, dim=-1)
            small = probs < 0.1 * probs.max(dim=-1, keepdim=True)[0]
            probs = torch.where(small, torch.full_like(probs, 1 / self.V), probs)
            logp = (probs / probs.sum(dim=-1, keepdim=True)).log()
        v = F.kl_div(logp, self.prev, reduction="none", log_target=True).sum(dim=-1)
        self.prev = logp
        return v < self.threshold, out, v


def generate_with_adaptive_compute(w, s: RavenShape, input_ids: torch.Tensor, max_new_tokens: int, criterion="none",
                                   exit_threshold="auto", num_steps=None, state_fn=None, continuous_compute=False,
                                   cache_lookup_strategy="full", do_not_exit_in_prefill=False, min_steps=0,
                                   check_criterion_every_n_steps=1, stop_tokens=(), init_scale=1.0, evaluator=None,
                                   record: Optional[dict] = None):
    """Greedy generate_with_adaptive_compute, RMM:1552-1749.  Every sequence of a batch keeps iterating until all
    have met the criterion (or max_steps); a sequence's logits are frozen at the step where it met it.
    `state_fn(call, shape)` supplies the initial latent state of each token step (call 0 is the prompt).
    Returns (ids, [per token: per sequence compute steps])."""
    cache = DictCache(cache_lookup_strategy)
    max_steps = s.mean_recurrence if num_steps is None else num_steps
    ids = input_ids.clone()
    B = ids.shape[0]
    draw = (lambda call, shape: state_fn(call, shape)) if state_fn is not None else \
        (lambda call, shape: initialize_state(torch.empty(shape), s, init_scale))
    carried = draw(0, (B, ids.shape[1], s.n_embd)) if continuous_compute else None      # RMM:1589-1591
    unfinished = torch.ones(B, dtype=torch.bool)
    ev = evaluator if evaluator is not None else ExitCriterion(criterion, exit_threshold, s.vocab_size)
    steps_log, values_log = [], []
    for token_step in range(max_new_tokens):
        seen = cache.get_seq_length()
        pos = torch.arange(seen, ids.shape[1])
        aux = dict(cache=cache, cache_position=pos)
        embeds, block_idx = embed_inputs(w, s, ids[:, pos], **aux)
        latents = carried if continuous_compute else draw(token_step, tuple(embeds.shape))
        if continuous_compute:
            next_states = latents[:, -1:, :].clone()
        predict = lambda lat: predict_from_latents(w, s, lat, **aux)
        steps_per_seq, values_per_seq = [0] * B, [[] for _ in range(B)]
        exit_reached = torch.zeros(B, dtype=torch.bool)
        outputs, next_logits = None, None
        ev.init(latents)
        broke = False
        for compute_step in range(max_steps):
            latents, block_idx = iterate_one_step(w, s, embeds, latents, block_idx, **aux)
            if (compute_step < min_steps or (compute_step - min_steps) % check_criterion_every_n_steps != 0
                    or (do_not_exit_in_prefill and token_step == 0)):
                continue
            new_exits, outputs, values = ev.check(latents, predict)
            for i in range(B):
                if not exit_reached[i] and unfinished[i]:
                    values_per_seq[i].append(float(values[i]))
            new_exits = new_exits & ~exit_reached & unfinished
            if new_exits.any():
                exit_reached = exit_reached | new_exits
                if outputs is None:
                    outputs = predict(latents)
                if next_logits is None:
                    next_logits = outputs.logits[:, -1, :].float().clone()
                else:
                    next_logits[new_exits] = outputs.logits[new_exits, -1, :].float()
                for i in range(B):
                    if new_exits[i]:
                        steps_per_seq[i] = compute_step + 1
                if continuous_compute:
                    next_states[new_exits] = latents[new_exits, -1:, :]
            if (exit_reached | ~unfinished).all():
                broke = True
                break
        if not broke:                                                                   # the loop's else branch
            if outputs is None:
                outputs = predict(latents)
            if next_logits is None:
                next_logits = outputs.logits[:, -1, :].float().clone()
                steps_per_seq = [max_steps] * B
            else:
                for i in range(B):
                    if not exit_reached[i] and unfinished[i]:
                        next_logits[i] = outputs.logits[i, -1, :].float()
                        steps_per_seq[i] = max_steps
        if continuous_compute:
            running = ~exit_reached & unfinished
            next_states[running] = latents[running, -1:, :]
            carried = next_states
        steps_log.append(steps_per_seq)
        values_log.append(values_per_seq)
        nxt = next_logits.argmax(dim=-1, keepdim=True)
        ids = torch.cat([ids, nxt], dim=-1)
        for i in range(B):
            if unfinished[i] and int(nxt[i, 0]) in stop_tokens:
                unfinished[i] = False
        if not unfinished.any():
            break
    if record is not None:
        record["cache"], record["exit_values"] = cache, values_log
    return ids, steps_log


def prefill_with_varied_exit_steps(w, s: RavenShape, input_ids: torch.Tensor, evaluator: ExitCriterion, state_fn=None,
                                   init_scale: float = 1.0, cache: Optional[DictCache] = None):
    """RMM:937-996: token by token, each token leaves the recurrence when the evaluator says so.
    Returns (logits [1, S, V], cache, compute steps per token)."""
    assert input_ids.shape[0] == 1
    cache = DictCache() if cache is None else cache
    rows, steps = [], []
    for p in range(input_ids.shape[1]):
        aux = dict(cache=cache, cache_position=torch.tensor([p]))
        embeds, block_idx = embed_inputs(w, s, input_ids[:, p:p + 1], **aux)
        latents = state_fn(p, tuple(embeds.shape)) if state_fn is not None else initialize_state(embeds, s, init_scale)
        evaluator.init(latents)
        predict = lambda lat: predict_from_latents(w, s, lat, **aux)
        step = -1
        for step in range(s.mean_recurrence):
            latents, block_idx = iterate_one_step(w, s, embeds, latents, block_idx, **aux)
            exits, _, _ = evaluator.check(latents, predict)
            if exits.any():
                break
        steps.append(step + 1)
        rows.append(predict(latents).logits)
    return torch.cat(rows, dim=1), cache, steps


def generate_speculative(w, s: RavenShape, input_ids: torch.Tensor, max_new_tokens: int, draft_steps: int, lookahead_for_draft: int,
                         num_steps: int, verification_threshold=1, state_fn=None, init_scale: float = 1.0,
                         continuous_compute=False, cache_lookup_strategy="full", stop_tokens=(), pad_id: int = 65509,
                         record: Optional[dict] = None):
    """Greedy generate_speculative, RMM:1750-1927: draft `lookahead_for_draft` tokens with `draft_steps` recurrences,
    drop them from the cache, verify all of them in one forward with `num_steps` recurrences, keep each sequence's
    agreeing prefix plus the verifier's own token at the first disagreement.  `state_fn(call, shape)` supplies the
    initial latent state of the call-th forward (prefill, drafts and verifications counted in order)."""
    assert lookahead_for_draft > 0
    L = lookahead_for_draft
    cache = DictCache(cache_lookup_strategy)
    ids = input_ids.clone()
    B = ids.shape[0]
    calls = [0]

    def run(tokens, pos, steps, carried):
        st = carried if carried is not None else (None if state_fn is None else state_fn(calls[0], (B, tokens.shape[1], s.n_embd)))
        calls[0] += 1
        return forward(w, s, input_ids=tokens, input_states=st, num_steps=steps, past_key_values=cache, use_cache=True,
                       cache_position=pos, init_scale=init_scale)

    carried = None
    if continuous_compute:                                              # RMM:1781-1783
        carried = state_fn(-1, (B, ids.shape[1], s.n_embd)) if state_fn is not None else \
            initialize_state(torch.empty(B, ids.shape[1], s.n_embd), s, init_scale)
    unfinished = torch.ones(B, dtype=torch.bool)
    generated = 0
    pos = torch.arange(0, ids.shape[1])
    out = run(ids, pos, num_steps, carried)                              # prefill with the full number of steps
    ids = torch.cat([ids, out.logits[:, -1, :].argmax(-1, keepdim=True)], dim=-1)
    generated += 1
    cache_position = torch.tensor([cache.get_seq_length()])
    if continuous_compute:
        carried = out.latent_states[:, -1:, :]
    prefix_len = ids.shape[1]
    accepted = []
    while generated < max_new_tokens:
        drafted = ids.clone()
        current_len = ids.shape[1]
        for _ in range(L):                                               # RMM:1809-1817
            out = run(drafted[:, cache_position], cache_position, draft_steps, carried)
            drafted = torch.cat([drafted, out.logits[:, -1, :].argmax(-1, keepdim=True)], dim=-1)
            cache_position = cache_position[-1:] + 1
            if continuous_compute:
                carried = out.latent_states[:, -1:, :]
        cache.clear_last_k_entries(L)
        cache_position = torch.arange(current_len - 1, current_len + L - 1)
        out = run(drafted[:, cache_position], cache_position, num_steps, carried)
        preds = out.logits.argmax(dim=-1)
        if verification_threshold >= 1:
            mismatched = preds[:, -L:] != drafted[:, current_len:]
            not_all, first_mismatch = torch.max(mismatched, dim=1)
        else:
            probs = F.softmax(out.logits[:, -L:, :], dim=-1)
            drafted_p = torch.gather(probs, -1, drafted[:, current_len:].unsqueeze(-1)).squeeze(-1)
            passed = drafted_p >= verification_threshold * probs.max(dim=-1)[0]
            not_all, first_mismatch = torch.max(~passed, dim=1)
        accept = torch.where(not_all, first_mismatch, L)
        per_seq = []
        for i in range(B):
            a = int(accept[i])
            if not_all[i] and a < L:
                final = out.logits[i:i + 1, a, :].argmax(-1, keepdim=True)
                part = drafted[i:i + 1, current_len:current_len + a]
                per_seq.append(torch.cat([part, final], dim=-1) if a > 0 else final)
            else:
                per_seq.append(drafted[i:i + 1, current_len:current_len + a])
        if not_all.any():
            cache.clear_last_k_entries(L - int(first_mismatch.min()) - 1)
        counts = [t.shape[1] for t in per_seq]
        width = max(counts)
        rows = [torch.cat([t, pad_id * torch.ones((1, width - t.shape[1]), dtype=t.dtype)], dim=-1) if t.shape[1] < width else t
                for t in per_seq]
        ids = torch.cat([ids, torch.cat(rows, dim=0)], dim=-1)
        accepted.append(counts)
        generated += width
        cache_position = torch.tensor([cache.get_seq_length()])
        if continuous_compute:
            carried = out.latent_states[:, -1:, :]
        for i in range(B):
            if unfinished[i] and any(int(t) in stop_tokens for t in per_seq[i].flatten()):
                unfinished[i] = False
        if not unfinished.any():
            break
    for i in range(B):                                                   # RMM:1903-1912: cut after the first stop token
        hits = [j for j, t in enumerate(ids[i, prefix_len:].tolist()) if t in stop_tokens]
        if hits:
            ids[i, prefix_len + hits[0] + 1:] = pad_id
    real = (ids != pad_id).any(dim=0).nonzero()
    if len(real) > 0:
        ids = ids[:, :int(real[-1]) + 1]
    if record is not None:
        record["accepted"], record["cache"], record["forwards"] = accepted, cache, calls[0]
    return ids


# --------------------------------------------------------------------------------------
# diffusion-style sampler (RMM:1234-1549): a wave of not-yet-frozen positions is re-run
# every step with a few recurrences, its cache entries are rolled back, positions freeze
# from the left
# --------------------------------------------------------------------------------------
def generate_diffusion_style(w, s: RavenShape, input_ids: torch.Tensor, max_new_tokens: int, *, num_steps: int = 32,
                             inner_recurrence: int = 4, headway: int = 1, freeze_strategy: str = "latent-diff",
                             exit_t: float = 0.03, ema_embeds: float = 0.1, state_noise_mixing: float = 0.5,
                             dampened_state_mixer: bool = True, sqrt_mixer: bool = False, continuous_compute: bool = False,
                             full_prefill: bool = True, max_wavefront: int = 128, max_diffusion_steps: int = 4096,
                             init_scale: float = 1.0, cache_lookup_strategy: str = "latest-m4-compress-s4", state_fn=None,
                             extra_token_fn=None, extra_token_high: int = 65510, stop_tokens=(), record: Optional[dict] = None):
    """Greedy generate_diffusion_style for one sequence.  `state_fn(draw, shape)` supplies the draw-th random latent state
    (the prefill's initial state, the first wave state, then per step the noise states and the states of new positions,
    in the order the loop draws them); `extra_token_fn(step, n)` the n = headway - 1 filler tokens of a step."""
    assert input_ids.shape[0] == 1, "one sequence"
    n_prompt, h = input_ids.shape[1], s.n_embd
    dt = w["transformer.wte.weight"].dtype
    cache = DictCache(cache_lookup_strategy)
    draws = [0]

    def draw(shape, via_bf16=False):
        x = state_fn(draws[0], shape) if state_fn is not None else initialize_state(torch.empty(shape), s, init_scale)
        draws[0] += 1
        # new positions and the prompt-wide wave are drawn from a bf16 template in the reference (RMM:1302, 1375-1378)
        return (x.to(torch.bfloat16) if via_bf16 else x).to(dt)

    width = max(s.block_size, n_prompt + max_new_tokens + headway + int(full_prefill))
    rec_count = torch.zeros(1, width, dtype=torch.long)   # recurrences spent per position
    stable = torch.zeros(1, width, dtype=torch.long)      # steps in which a position's token did not change
    passes = tokens_forward = clears = standing = 0

    if full_prefill:                                                      # RMM:1289-1299
        out = forward(w, s, input_ids=input_ids, input_states=draw((1, n_prompt, h)), num_steps=num_steps, past_key_values=cache,
                      use_cache=True, cache_position=torch.arange(n_prompt), init_scale=init_scale)
        passes, tokens_forward = passes + 1, tokens_forward + n_prompt
        frozen = current = torch.cat([input_ids, out.logits[:, -1, :].argmax(-1, keepdim=True)], dim=-1)
        rec_count[:, :frozen.shape[1]] += num_steps
        states = draw((1, 1, h))
    else:                                                                 # RMM:1300-1309
        states = draw((1, n_prompt, h), via_bf16=True)
        frozen, current = input_ids.clone(), input_ids.clone()
        if 0 < max_wavefront < states.shape[1]:
            raise ValueError("prompt longer than max_wavefront: use full_prefill")

    if ema_embeds > 0.0:
        old_embeds, _ = embed_inputs(w, s, current)                        # without a cache (RMM:1311-1312)
    latent = "latent" in freeze_strategy
    accel = "latent-acceleration" in freeze_strategy
    if latent:
        prev_states = states.clone()
    if accel:
        prev_delta, prev_prev_states, old_old_ci = torch.zeros_like(states), torch.zeros_like(states), 0
    old_ci, old_k, k, step = 0, 0, 0, 0
    log = []

    while frozen.shape[1] - n_prompt < max_new_tokens and current.shape[1] <= s.block_size:
        ci = cache.get_seq_length()
        n_wave = states.shape[1]
        pos = torch.arange(ci, ci + n_wave)
        new_embeds, block_idx = embed_inputs(w, s, current[:, pos], cache=cache, cache_position=pos)
        if ema_embeds > 0.0:                                               # RMM:1337-1342
            carry = old_embeds[:, ci - old_ci:]
            embeds = new_embeds.clone() * (1 - ema_embeds)
            embeds[:, :carry.shape[1], :] += carry * ema_embeds
            old_embeds = embeds.clone()
        else:
            embeds = new_embeds
        if state_noise_mixing > 0:                                         # RMM:1346-1357
            noise_states = draw(tuple(states.shape))
            if dampened_state_mixer:
                mix = (state_noise_mixing / (1 + rec_count[:, ci:ci + n_wave]))[:, :, None].to(states.dtype)
            else:
                mix = torch.as_tensor(state_noise_mixing, dtype=states.dtype)
            if sqrt_mixer:
                states = states * F.relu(1 - mix).sqrt() + mix.sqrt() * noise_states
            else:
                states = states * (1 - mix) + mix * noise_states
        for _ in range(inner_recurrence):                                  # RMM:1358-1362
            states, block_idx = iterate_one_step(w, s, embeds, states, block_idx, cache=cache, cache_position=pos)
            rec_count[:, ci:ci + n_wave] += 1
            passes, tokens_forward = passes + 1, tokens_forward + n_wave
        logits = predict_from_latents(w, s, states, cache=cache, cache_position=pos).logits
        first_state, first_logits = states[0, 0].clone(), logits[0, 0].clone()  # of the wave's leftmost position, for the record
        wave_states = states[0].clone()                                         # of every position of the wave
        # positions whose prediction is not frozen yet: from the last frozen token on (RMM:1366-1369)
        new_tokens = logits[0, max(frozen.shape[1] - 1 - ci, 0):, :].argmax(-1, keepdim=True).T
        guess = torch.cat([frozen, new_tokens[:, :-1]], dim=1)
        stable[:, :current.shape[1]] += current == guess
        if extra_token_fn is not None:
            extra = extra_token_fn(step, headway - 1).view(1, headway - 1)
        else:
            extra = torch.randint(0, extra_token_high, (1, headway - 1))
        current = torch.cat([frozen, new_tokens, extra], dim=1)
        if continuous_compute and states.shape[1] >= headway:
            fresh = states[:, -headway:].clone()
        else:
            fresh = draw((1, headway, h), via_bf16=True)
        states = torch.cat([states, fresh], dim=1)
        headway_now = headway
        if max_wavefront > 0 and states.shape[1] > max_wavefront:          # RMM:1384-1394: the wave stops growing
            headway_now = max_wavefront - (states.shape[1] - headway)
            states = states[:, :max_wavefront]
            current = current[:, :ci + max_wavefront]
            standing += 1

        def freeze_up_to(k_new):                                           # RMM:1437-1444 and its two siblings
            nonlocal states, frozen, clears
            n_clear = current.shape[1] - headway_now - k_new + 1
            cache.clear_last_k_entries(n_clear)
            clears += n_clear
            states = states[:, k_new - ci - 1:, :]
            frozen = current[:, :k_new]

        def freeze_nothing():
            nonlocal clears
            cache.clear_last_k_entries(states.shape[1] - headway_now)
            clears += states.shape[1] - headway_now

        if latent:
            if freeze_strategy == "latent-diff":                           # RMM:1396-1400
                old = prev_states[:, ci - old_ci:]
                cur = states[:, :old.shape[1], :]
                criterion = (cur - old).norm(dim=-1) / cur.norm(dim=-1)
            elif freeze_strategy == "latent-acceleration-1":               # RMM:1401-1412
                old = prev_states[:, ci - old_ci:]
                cur = states[:, :old.shape[1], :]
                delta = cur - old
                m = min(delta.shape[1], prev_delta.shape[1])
                criterion = (delta[:, :m, :] - prev_delta[:, :m, :]).norm(dim=-1) / cur[:, :m, :].norm(dim=-1)
                prev_delta = delta.clone()
            elif freeze_strategy == "latent-acceleration-2":               # RMM:1414-1435
                lo = max(ci, old_ci, old_old_ci)
                hi = min(ci + states.shape[1], old_ci + prev_states.shape[1], old_old_ci + prev_prev_states.shape[1])
                a, b, c = states[:, lo - ci:hi - ci], prev_states[:, lo - old_ci:hi - old_ci], \
                    prev_prev_states[:, lo - old_old_ci:hi - old_old_ci]
                criterion = ((a - b) - (b - c)).norm(dim=-1) / (a.norm(dim=-1) + 1e-6)
            else:
                raise ValueError(freeze_strategy)
            exits = criterion < exit_t
            if exits.sum() > 0:
                k = ci + int(exits.nonzero()[-1][1]) + 1
                freeze_up_to(k)
            else:
                freeze_nothing()
        elif freeze_strategy == "token-stability":                         # RMM:1450-1463
            ripe = stable > num_steps // inner_recurrence
            if torch.any(ripe):
                k = int(ripe.nonzero()[-1][1]) + 1
                freeze_up_to(k)
            else:
                freeze_nothing()
                k = 0
        elif freeze_strategy == "fixed":                                   # RMM:1464-1474
            if step > num_steps // inner_recurrence:
                n_clear = states.shape[1] - headway - headway_now
                cache.clear_last_k_entries(n_clear)
                clears += n_clear
                states = states[:, headway_now:, :]
                frozen = torch.cat([frozen, new_tokens[:, :headway_now]], dim=-1)
            else:
                freeze_nothing()
        else:
            raise ValueError(f"Invalid freeze strategy {freeze_strategy}")
        log.append(dict(step=step, cache_index=ci, wave=n_wave, frozen=frozen.shape[1], current=current[0].tolist(),
                        first_state=first_state, first_logits=first_logits, wave_states=wave_states, wave_logits=logits[0].clone()))

        if step > num_steps:                                               # RMM:1478-1492
            seen = frozen[0, old_k:k].tolist() if latent else frozen[0, -headway:].tolist()
            if any(t in stop_tokens for t in seen):
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

    if record is not None:
        record.update(num_core_forward_passes=passes, num_tokens_forward=tokens_forward, num_cache_clears=clears,
                      num_standing_waves=standing, diffusion_steps=step, gen_seq_length=current.shape[1], len_prefill=n_prompt,
                      recurrence_per_position=rec_count[:, :frozen.shape[1]].clone(),
                      token_stable_per_position=stable[:, :frozen.shape[1]].clone(), cache=cache, log=log, draws=draws[0])
    return frozen


# --------------------------------------------------------------------------------------
# closed-form accounting used as known-answer tests and by the roofline arithmetic
# --------------------------------------------------------------------------------------
def n_cache_slots(s: RavenShape, num_steps: Optional[int] = None) -> int:
    r = s.mean_recurrence if num_steps is None else num_steps
    return s.n_layers_in_prelude + s.n_layers_in_recurrent_block * r + s.n_layers_in_coda


def step_indices(s: RavenShape, num_steps: Optional[int] = None) -> list[int]:
    """Order in which one forward touches the cache slots (RMM:677-681, 774-779, 697-700)."""
    r = s.mean_recurrence if num_steps is None else num_steps
    idx = list(range(s.n_layers_in_prelude + s.n_layers_in_recurrent_block * r))
    return idx + [-(i + 1) for i in range(s.n_layers_in_coda)]


def core_iteration_bytes(s: RavenShape, batch: int, t_cached: int, elt: int = 2) -> dict:
    """Algorithmic HBM bytes of one recurrence iteration at decode: weights once, KV read, KV write."""
    h, inter, nb = s.n_embd, s.intermediate_size, s.n_layers_in_recurrent_block
    per_block = (3 * h * h + h * h + 2 * inter * h + h * inter + 4 * h + (2 * h if s.qk_bias else 0)) * elt
    weights = nb * per_block + 2 * h * h * elt
    kv_read = batch * nb * 2 * h * t_cached * elt
    kv_write = batch * nb * 2 * h * elt
    return {"weights": weights, "kv_read": kv_read, "kv_write": kv_write, "total": weights + kv_read + kv_write}
