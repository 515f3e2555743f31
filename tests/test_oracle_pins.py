"""Pins for the CPU oracle: each check is something the mathematics or a library routine fixes
independently of the oracle's own formulas, chosen so that a dropped term, a wrong sign or index,
or a swapped operand fails at least one of them.  The reference holds no golden vectors for this
path; its only exact published numbers (three KV-cache sizes, examples/inference_demo.ipynb:252,
373, 491) are used as known-answer tests at the bottom."""

import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import raven_oracle as O

torch.manual_seed(1234)
EPS = 1e-6


# ----------------------------------------------------------------------------- RMSNorm
def test_rmsnorm_constant_row_closed_form():
    n, c = 5280, 3.0
    w = torch.linspace(0.5, 1.5, n)
    y = O.rmsnorm(torch.full((2, n), c), w, EPS)
    assert torch.allclose(y, w * c / math.sqrt(c * c + EPS), rtol=1e-6, atol=0)


def test_rmsnorm_one_hot_row_closed_form():
    n, c, j = 96, -2.5, 17
    x = torch.zeros(1, n)
    x[0, j] = c
    w = torch.rand(n) + 0.5
    y = O.rmsnorm(x, w, EPS)
    assert y[0, j].item() == pytest.approx(w[j].item() * c / math.sqrt(c * c / n + EPS), rel=1e-6)
    assert y[0].abs().sum().item() == pytest.approx(abs(y[0, j].item()), rel=1e-6)


def test_rmsnorm_brute_force_fp64_and_library():
    x = torch.randn(5, 16)
    w = torch.randn(16)
    want = torch.empty(5, 16, dtype=torch.float64)
    for i in range(5):
        ms = sum(float(v) ** 2 for v in x[i]) / 16
        for j in range(16):
            want[i, j] = float(x[i, j]) / math.sqrt(ms + EPS) * float(w[j])
    assert torch.allclose(O.rmsnorm(x, w, EPS).double(), want, rtol=1e-5, atol=1e-6)
    lib = F.rms_norm(x, (16,), eps=EPS) * w
    assert torch.allclose(O.rmsnorm(x, w, EPS), lib, rtol=1e-5, atol=1e-6)


def test_rmsnorm_scale_invariance_and_eps_placement():
    x = torch.randn(3, 256)
    w = torch.ones(256)
    assert torch.allclose(O.rmsnorm(x, w, EPS), O.rmsnorm(1000.0 * x, w, EPS), rtol=1e-4, atol=1e-5)
    # eps is added to the MEAN of squares (not the sum, not outside the sqrt): tiny inputs expose it
    tiny = torch.full((1, 4), 1e-3)
    assert O.rmsnorm(tiny, torch.ones(4), 1e-6)[0, 0].item() == pytest.approx(1e-3 / math.sqrt(2e-6), rel=1e-5)


def test_rmsnorm_rounds_before_weight_in_bf16():
    x = torch.randn(64, 5280).bfloat16()
    w = (1 + 0.02 * torch.randn(5280)).bfloat16()
    got = O.rmsnorm(x, w, EPS)
    x32 = x.float()
    normed = x32 * torch.rsqrt((x32 * x32).mean(-1, keepdim=True) + EPS)
    two_roundings = (normed.bfloat16().float() * w.float()).bfloat16()
    one_rounding = (normed * w.float()).bfloat16()
    assert got.dtype == torch.bfloat16
    assert torch.equal(got, two_roundings)
    assert not torch.equal(two_roundings, one_rounding)  # the distinction is observable


# ----------------------------------------------------------------------------- RoPE
def test_rope_table_spot_values_and_shape():
    t = O.rope_table(96, 4096, 50000.0)
    assert t.shape == (1, 4096, 1, 48, 2) and t.dtype == torch.float32
    for pos, i in [(0, 0), (1, 0), (7, 5), (1023, 47), (4095, 13)]:
        ang = np.float32(pos) * np.float32(1.0 / (50000.0 ** (2 * i / 96)))
        assert t[0, pos, 0, i, 0].item() == pytest.approx(math.cos(ang), abs=2e-4)
        assert t[0, pos, 0, i, 1].item() == pytest.approx(math.sin(ang), abs=2e-4)
    assert torch.equal(t[0, 0, 0, :, 0], torch.ones(48)) and torch.equal(t[0, 0, 0, :, 1], torch.zeros(48))


def test_rope_equals_complex_multiplication():
    b, s, nh, hd = 2, 5, 3, 8
    q, k = torch.randn(b, s, nh, hd), torch.randn(b, s, nh, hd)
    tab = O.rope_table(hd, 16, 50000.0)[:, 3:3 + s]
    rq, rk = O.apply_rope(q, k, tab)
    ang = torch.outer(torch.arange(3, 3 + s).float(), 1.0 / (50000.0 ** (torch.arange(0, hd, 2).float() / hd)))
    cis = torch.polar(torch.ones_like(ang), ang)[None, :, None, :]
    for got, src in ((rq, q), (rk, k)):
        want = torch.view_as_real(torch.view_as_complex(src.reshape(b, s, nh, hd // 2, 2)) * cis).flatten(3)
        assert torch.allclose(got, want, rtol=1e-5, atol=1e-6)


def test_rope_identity_norm_and_relative_position():
    hd = 96
    tab = O.rope_table(hd, 64, 50000.0)
    q, k = torch.randn(1, 1, 2, hd), torch.randn(1, 1, 2, hd)
    q0, k0 = O.apply_rope(q, k, tab[:, 0:1])
    assert torch.equal(q0, q) and torch.equal(k0, k)
    qm, _ = O.apply_rope(q, k, tab[:, 9:10])
    pn = lambda t: t.unflatten(-1, (-1, 2)).norm(dim=-1)
    assert torch.allclose(pn(qm), pn(q), rtol=1e-5, atol=1e-6)
    dots = []
    for m, n in ((9, 4), (25, 20), (45, 40)):
        a, _ = O.apply_rope(q, q, tab[:, m:m + 1])
        _, c = O.apply_rope(k, k, tab[:, n:n + 1])
        dots.append((a * c).sum().item())
    assert dots[0] == pytest.approx(dots[1], rel=1e-4, abs=1e-4) and dots[1] == pytest.approx(dots[2], rel=1e-4, abs=1e-4)
    # sign convention: rotating (1, 0) by +angle gives (cos, +sin)
    e = torch.zeros(1, 1, 1, hd)
    e[..., 0] = 1.0
    r, _ = O.apply_rope(e, e, tab[:, 5:6])
    assert r[0, 0, 0, 0].item() == pytest.approx(math.cos(5.0), abs=1e-5)
    assert r[0, 0, 0, 1].item() == pytest.approx(math.sin(5.0), abs=1e-5)


# ----------------------------------------------------------------------------- attention
def _eager64(q, k, v, mask=None):
    s = (q.double() @ k.double().transpose(-1, -2)) / math.sqrt(q.shape[-1])
    if mask is not None:
        s = s.masked_fill(~mask, float("-inf"))
    return torch.softmax(s, -1) @ v.double()


def test_sdpa_decode_special_cases():
    q, k, v = torch.randn(2, 3, 1, 16), torch.randn(2, 3, 7, 16), torch.randn(2, 3, 7, 16)
    assert torch.allclose(O.sdpa(q, k, v).double(), _eager64(q, k, v), rtol=1e-5, atol=1e-6)
    assert torch.allclose(O.sdpa(q, k[..., :1, :], v[..., :1, :]), v[..., :1, :], rtol=1e-6, atol=1e-7)
    assert torch.allclose(O.sdpa(torch.zeros_like(q), k, v), v.mean(-2, keepdim=True), rtol=1e-5, atol=1e-6)


def test_sdpa_mask_cases_match_library():
    q, k, v = torch.randn(1, 2, 5, 8), torch.randn(1, 2, 5, 8), torch.randn(1, 2, 5, 8)
    assert torch.allclose(O.sdpa(q, k, v), F.scaled_dot_product_attention(q, k, v, is_causal=True), rtol=1e-5, atol=1e-6)
    k2, v2 = torch.randn(1, 2, 9, 8), torch.randn(1, 2, 9, 8)
    mask = torch.ones(5, 9, dtype=torch.bool).tril(diagonal=4)       # lower-right aligned causal
    assert torch.allclose(O.sdpa(q, k2, v2).double(), _eager64(q, k2, v2, mask), rtol=1e-5, atol=1e-6)
    lib = F.scaled_dot_product_attention(q, k2, v2, attn_mask=mask)
    assert torch.allclose(O.sdpa(q, k2, v2), lib, rtol=1e-5, atol=1e-6)
    q1 = q[..., :1, :]
    assert torch.allclose(O.sdpa(q1, k2, v2), F.scaled_dot_product_attention(q1, k2, v2), rtol=1e-5, atol=1e-6)


# ----------------------------------------------------------------------------- linear pieces
def _tiny(dtype=torch.float32, seed=0):
    s = O.RavenShape.tiny()
    return s, O.make_weights(s, seed=seed, dtype=dtype)


def test_adapter_operand_order_and_split_identity():
    s, w = _tiny()
    h = s.n_embd
    state, emb = torch.randn(1, 1, h), torch.randn(1, 1, h)
    wa = w["transformer.adapter.weight"]
    want = (state.double() @ wa[:, :h].double().T) + (emb.double() @ wa[:, h:].double().T)
    blocks_off = dict(w)
    got = F.linear(torch.cat([state, emb], -1), wa)
    assert torch.allclose(got.double(), want, rtol=1e-5, atol=1e-6)
    swapped = F.linear(torch.cat([emb, state], -1), wa)
    assert not torch.allclose(got, swapped, rtol=1e-3, atol=1e-4)
    # the oracle's core step applies exactly that adapter before its blocks
    s0 = O.RavenShape(**{**s.__dict__, "n_layers_in_recurrent_block": 0})
    x, idx = O.core_block_forward(state, emb, blocks_off, None, None, 0, s0)
    assert torch.equal(x, got) and idx == 0


def test_gated_mlp_fp64_and_gate_half():
    s, w = _tiny()
    p = "transformer.core_block.0"
    x = torch.randn(2, 3, s.n_embd)
    fc, pr = w[f"{p}.mlp.fc.weight"].double(), w[f"{p}.mlp.proj.weight"].double()
    z = x.double() @ fc.T
    a, b = z[..., : s.intermediate_size], z[..., s.intermediate_size:]
    want = ((a / (1 + torch.exp(-a))) * b) @ pr.T
    got = O.gated_mlp(x, w, p).double()
    assert torch.allclose(got, want, rtol=1e-4, atol=1e-7)
    wrong = ((b / (1 + torch.exp(-b))) * a) @ pr.T
    assert not torch.allclose(got, wrong, rtol=1e-2, atol=1e-5)


def test_attention_projection_split_bias_and_cache_contents():
    s, w = _tiny()
    p = "transformer.prelude.0"
    h, nh, hd = s.n_embd, s.n_heads, s.head_dim
    x = torch.randn(2, 3, h)
    freqs = w["freqs_cis"][:, 4:7]
    cache = O.DictCache()
    cache._seen_tokens = 4  # pretend four tokens were seen; step 0 adds 3 more
    out = O.attention(x, w, p, freqs, 0, cache, s)
    qkv = x.double() @ w[f"{p}.attn.Wqkv.weight"].double().T
    q, k, v = qkv[..., :h], qkv[..., h:2 * h], qkv[..., 2 * h:]
    bias = w[f"{p}.attn.qk_bias"].double()
    k = (k.view(2, 3, nh, hd) + bias[1])
    ang = torch.outer(torch.arange(4, 7).double(), 1.0 / (50000.0 ** (torch.arange(0, hd, 2).double() / hd)))
    cis = torch.polar(torch.ones_like(ang), ang)[None, :, None, :]
    k_rot = torch.view_as_real(torch.view_as_complex(k.reshape(2, 3, nh, hd // 2, 2).contiguous()) * cis).flatten(3)
    assert sorted(cache.key_cache[0]) == [4, 5, 6] and cache.get_seq_length() == 7
    for i, pos in enumerate((4, 5, 6)):
        assert torch.allclose(cache.key_cache[0][pos].double(), k_rot[:, i], rtol=1e-4, atol=1e-5)  # post-bias, post-RoPE
        assert torch.allclose(cache.value_cache[0][pos].double(), v.view(2, 3, nh, hd)[:, i], rtol=1e-4, atol=1e-5)  # no bias on v
    assert out.shape == (2, 3, h)


def test_sandwich_block_is_the_stated_composition():
    s, w = _tiny()
    p = "transformer.core_block.1"
    x = torch.randn(1, 4, s.n_embd)
    freqs = w["freqs_cis"][:, :4]
    got = O.sandwich_block(x, w, p, freqs, 3, None, s)
    n = lambda t, k: O.rmsnorm(t, w[f"{p}.norm_{k}.weight"], s.norm_eps)
    a = O.attention(n(x, 1), w, p, freqs, 3, None, s)
    x2 = n(a + x, 2)
    want = n(O.gated_mlp(n(x2, 3), w, p) + x2, 4)
    assert torch.equal(got, want)
    # a residual taken from the wrong place (pre-norm style) gives something else
    wrong = n(O.gated_mlp(n(x2, 3), w, p) + x, 4)
    assert not torch.allclose(got, wrong, rtol=1e-3, atol=1e-4)


# ----------------------------------------------------------------------------- recurrence and forward
def test_num_steps_forms_and_zero_steps():
    s, w = _tiny()
    emb = torch.randn(1, 2, s.n_embd)
    st = torch.randn(1, 2, s.n_embd)
    fr = w["freqs_cis"][:, :2]
    y0, idx0 = O.iterate_forward(emb, st, w, fr, 0, None, 0, s)
    assert torch.equal(y0, O.rmsnorm(st, w["transformer.ln_f.weight"], s.norm_eps)) and idx0 == 0
    a, ia = O.iterate_forward(emb, st, w, fr, 0, None, 3, s)
    b, ib = O.iterate_forward(emb, st, w, fr, 0, None, torch.tensor(3), s)
    c, ic = O.iterate_forward(emb, st, w, fr, 0, None, (2, 1), s)
    d, idd = O.iterate_forward(emb, st, w, fr, 0, None, None, O.RavenShape(**{**s.__dict__, "mean_recurrence": 3}))
    assert torch.equal(a, b) and torch.equal(a, c) and torch.equal(a, d)
    assert ia == ib == ic == idd == 3 * s.n_layers_in_recurrent_block


def test_step_index_enumeration():
    assert O.step_indices(O.RavenShape.nebel()) == list(range(130)) + [-1, -2]
    assert O.step_indices(O.RavenShape.tiny()) == list(range(9)) + [-1]
    assert O.n_cache_slots(O.RavenShape.nebel()) == 132
    s, w = _tiny()
    cache = O.DictCache()
    O.forward(w, s, input_ids=torch.randint(0, s.vocab_size, (1, 3)), input_states=torch.zeros(1, 3, s.n_embd),
              past_key_values=cache, use_cache=True)
    assert list(cache.key_cache) == O.step_indices(s)
    assert all(sorted(c) == [0, 1, 2] for c in cache.key_cache.values())
    assert cache.get_seq_length() == 3


def test_cache_and_no_cache_agree_and_prefill_then_decode():
    s, w = _tiny()
    ids = torch.randint(0, s.vocab_size, (2, 6))
    states = 0.6 * torch.randn(2, 6, s.n_embd)
    full = O.forward(w, s, input_ids=ids, input_states=states).logits
    # prefill 4, then two single-token decode steps through the cache
    cache = O.DictCache()
    a = O.forward(w, s, input_ids=ids[:, :4], input_states=states[:, :4], past_key_values=cache, use_cache=True,
                  cache_position=torch.arange(0, 4)).logits
    b = O.forward(w, s, input_ids=ids[:, 4:5], input_states=states[:, 4:5], past_key_values=cache, use_cache=True,
                  cache_position=torch.arange(4, 5)).logits
    c = O.forward(w, s, input_ids=ids[:, 5:6], input_states=states[:, 5:6], past_key_values=cache, use_cache=True,
                  cache_position=torch.arange(5, 6)).logits
    got = torch.cat([a, b, c], dim=1)
    assert torch.allclose(got, full, rtol=1e-4, atol=1e-5)
    # two-token chunk against a longer cache exercises the lower-right-aligned causal case
    cache2 = O.DictCache()
    O.forward(w, s, input_ids=ids[:, :4], input_states=states[:, :4], past_key_values=cache2, use_cache=True,
              cache_position=torch.arange(0, 4))
    d = O.forward(w, s, input_ids=ids[:, 4:6], input_states=states[:, 4:6], past_key_values=cache2, use_cache=True,
                  cache_position=torch.arange(4, 6)).logits
    assert torch.allclose(d, full[:, 4:6], rtol=1e-4, atol=1e-5)


def test_forward_head_is_tied_scaled_and_double_normed():
    s, w = _tiny()
    ids = torch.randint(0, s.vocab_size, (1, 2))
    st = torch.randn(1, 2, s.n_embd)
    out = O.forward(w, s, input_ids=ids, input_states=st, num_steps=0)
    # with zero recurrences the latent is ln_f(state), and the logits follow from the coda alone
    lat = O.rmsnorm(st, w["transformer.ln_f.weight"], s.norm_eps)
    assert torch.equal(out.latent_states, lat)
    x = O.sandwich_block(lat, w, "transformer.coda.0", w["freqs_cis"][:, :2], -1, None, s)
    x = O.rmsnorm(x, w["transformer.ln_f.weight"], s.norm_eps)
    assert torch.allclose(out.logits, x @ w["transformer.wte.weight"].T, rtol=1e-5, atol=1e-6)
    assert out.logits.dtype == torch.float32
    # embedding scale sqrt(n_embd): feeding pre-scaled embeddings by hand must not change anything
    emb = F.embedding(ids, w["transformer.wte.weight"])
    out2 = O.forward(w, s, input_embeds=emb, input_states=st, num_steps=1)
    out3 = O.forward(w, s, input_ids=ids, input_states=st, num_steps=1)
    assert torch.equal(out2.logits, out3.logits)
    pre = O.sandwich_block(emb * 16.0, w, "transformer.prelude.0", w["freqs_cis"][:, :2], 0, None, s)
    x1, _ = O.core_block_forward(st, pre, w, w["freqs_cis"][:, :2], None, 0, s)
    assert torch.equal(out3.latent_states, O.rmsnorm(x1, w["transformer.ln_f.weight"], s.norm_eps))


def test_initialize_state_distribution():
    s = O.RavenShape.nebel()
    g = torch.Generator().manual_seed(7)
    x = O.initialize_state(torch.empty(4, 8, s.n_embd), s, 1.0, g)
    bound = 3 * s.init_std * s.emb_scale
    assert x.abs().max().item() <= bound * (1 + 1e-6)
    assert x.std().item() == pytest.approx(math.sqrt(2 / 5) * 0.9866, rel=2e-2)  # std of a +-3 sigma truncated normal
    assert torch.equal(x, O.initialize_state(torch.empty(4, 8, s.n_embd), s, 1.0, torch.Generator().manual_seed(7)))
    assert O.initialize_state(torch.empty(1, 2, 16), s, 0.0).abs().sum().item() == 0.0


def test_greedy_is_argmax_of_last_position_and_deterministic():
    s, w = _tiny()
    prompt = torch.randint(0, s.vocab_size, (1, 8), generator=torch.Generator().manual_seed(3))
    rec = {}
    ids = O.greedy_generate(w, s, prompt, 5, record=rec)
    assert ids.shape == (1, 13) and torch.equal(ids[:, :8], prompt)
    ids2 = O.greedy_generate(w, s, prompt, 5)
    assert torch.equal(ids, ids2)
    # first new token equals argmax of a cache-less full forward with a zero state
    logits = O.forward(w, s, input_ids=prompt, input_states=torch.zeros(1, 8, s.n_embd)).logits
    assert int(ids[0, 8]) == int(logits[0, -1].argmax())
    assert rec["cache"].get_seq_length() == 12  # the last generated token was never fed back
    assert len(rec["margins"]) == 5


# ----------------------------------------------------------------------------- cache model
def test_dict_cache_against_list_model():
    rng = torch.Generator().manual_seed(5)
    cache = O.DictCache()
    log: dict[int, list] = {}
    seen = 0
    for n_new in (3, 1, 1, 2):
        for step in (0, 1, 2, 5, -1):
            k = torch.randn(2, 3, n_new, 4, generator=rng)
            v = torch.randn(2, 3, n_new, 4, generator=rng)
            if step == 0:
                seen += n_new
            log.setdefault(step, []).append((k, v))
            gk, gv = cache.update(k, v, torch.tensor(step))
            assert torch.equal(gk, torch.cat([a for a, _ in log[step]], dim=-2))
            assert torch.equal(gv, torch.cat([b for _, b in log[step]], dim=-2))
            assert cache.get_seq_length() == seen
    assert seen == 7 and sorted(cache.key_cache[5]) == list(range(7))
    cache.clear_last_k_entries(2)
    assert cache.get_seq_length() == 5 and all(sorted(c) == list(range(5)) for c in cache.key_cache.values())
    with pytest.raises(AssertionError):
        cache.update(torch.zeros(2, 3, 1, 4), torch.zeros(2, 3, 1, 4), 1)  # step 1 before step 0: position 4 exists
    cache.reset()
    assert cache.get_seq_length() == 0 and not cache.key_cache


def test_partial_fill_lookups_closed_form():
    """Tokens with different numbers of recurrences: entries are tagged with (step, position), so what a lookup
    returns names its source.  For a token that ran d recurrences, block j of recurrence i (step 2 + 4i + j) must come
    from recurrence min(i, d - 1) under latest-m4 / available-m4, from recurrence d - 1 under always-last-m4 whenever
    the step has a gap at all, and is dropped by skip / full when i >= d (RMM:199-253)."""
    depths = [3, 1, 4, 2, 5]  # recurrences per token; the querying token runs 5
    for strategy in ("latest-m4", "available-m4", "always-last-m4", "skip", "full"):
        c = O.DictCache(strategy)
        for pos, d in enumerate(depths):
            for step in [0, 1] + list(range(2, 2 + 4 * d)):
                tag = torch.full((1, 1, 1, 1), float(step * 100 + pos))
                k, _ = c.update(tag, tag, step)
                got = [(int(t) // 100, int(t) % 100) for t in k.flatten().tolist()]
                if step < 2:
                    assert got == [(step, p) for p in range(pos + 1)]
                    continue
                i, j = divmod(step - 2, 4)
                older = depths[:pos]
                gap = any(dd <= i for dd in older)
                want = []
                for p, dd in enumerate(older):
                    if not gap or (strategy in ("latest-m4", "available-m4") and i < dd):
                        want.append((step, p))
                    elif strategy in ("skip", "full"):
                        if i < dd:
                            want.append((step, p))
                    elif strategy == "always-last-m4":
                        want.append((2 + 4 * (dd - 1) + j, p))
                    else:
                        want.append((2 + 4 * min(i, dd - 1) + j, p))
                want.append((step, pos))
                assert got == want, (strategy, pos, step, got, want)


def test_randomized_lookup_draws_one_step_per_position():
    """RMM:255-271: once a step has a gap, every position (the querying one too) is read at a step of the same block,
    not deeper than the current step, drawn among those it holds -- one draw of `torch.randint(n_valid, (1,))` per
    position, in position order, from the CPU's default generator.  Entries are tagged with (step, position); the draws
    are replayed from the same seed, and the generator must stand where the replay leaves it."""
    depths = [3, 1, 4, 2, 5]
    seen_choices = set()
    for seed in range(6):
        c = O.DictCache("randomized")
        for pos, d in enumerate(depths):
            for step in [0, 1] + list(range(2, 2 + 4 * d)):
                tag = torch.full((1, 1, 1, 1), float(step * 100 + pos))
                torch.manual_seed(1000 * seed + 10 * pos + step)
                k, _ = c.update(tag, tag, step)
                after = int(torch.randint(1 << 30, (1,)))
                got = [(int(t) // 100, int(t) % 100) for t in k.flatten().tolist()]
                if step < 2 or all(dd > (step - 2) // 4 for dd in depths[:pos]):
                    assert got == [(step, p) for p in range(pos + 1)]  # no gap: no draw
                    continue
                i, j = divmod(step - 2, 4)
                torch.manual_seed(1000 * seed + 10 * pos + step)
                want = []
                for p, dd in enumerate(depths[:pos] + [i + 1]):
                    n_valid = min(i + 1, dd)
                    want.append((2 + 4 * int(torch.randint(n_valid, (1,))) + j, p))
                assert got == want, (seed, pos, step, got, want)
                assert after == int(torch.randint(1 << 30, (1,)))
                seen_choices.update((pos, step, src) for src, p in got if p == 2)
    # position 2 holds 4 recurrences: queried at recurrence 4 (step 18..21, token 4) each of its four is drawn at some seed
    assert {src for pos, step, src in seen_choices if step == 18} == {2, 6, 10, 14}


def test_step_remap_strategies():
    assert [O.remap_step(i, "full") for i in (0, 1, 2, 129, -1)] == [0, 1, 2, 129, -1]
    assert [O.remap_step(i, "latest-m4-compress-s4") for i in (0, 1, 2, 5, 6, 9, 129, -1, -2)] == [0, 1, 2, 5, 2, 5, 5, -1, -2]
    assert [O.remap_step(i, "compress-s16") for i in (2, 17, 18, 33, 34)] == [2, 17, 2, 17, 2]
    assert [O.remap_step(i, "compress-r4") for i in (2, 5, 6, 129)] == [2, 2, 3, 33]
    assert [O.remap_step(i, "compress-anchor") for i in (2, 33, 34, 37, 38, 41, 129)] == [2, 33, 34, 37, 34, 37, 37]


def test_published_cache_sizes():
    """examples/inference_demo.ipynb:252, 373, 491 of the reference."""
    s = O.RavenShape.nebel()
    entry = torch.zeros(1, s.n_heads, s.head_dim, dtype=torch.bfloat16)
    c = O.DictCache()
    for step in O.step_indices(s):
        c.key_cache[step] = {p: entry for p in range(366)}
    assert c.get_memory_usage() == 973.0810546875
    c16 = O.DictCache("latest-m4-compress-s16")
    for step in sorted({O.remap_step(i, c16.lookup_strategy) for i in O.step_indices(s)}):
        c16.key_cache[step] = {p: entry for p in range(366)}
    assert len(c16.key_cache) == 20 and c16.get_memory_usage() == 147.4365234375
    assert 132 * 55 * 1024 * 96 * 2 * 2 / 2**20 == 2722.5


def test_core_iteration_byte_count_at_the_3_5b_shape():
    s = O.RavenShape.nebel()
    b1 = O.core_iteration_bytes(s, 1, 1024)
    assert b1["weights"] == 3_274_698_240 and b1["kv_read"] == 86_507_520 and b1["kv_write"] == 84_480
    assert O.core_iteration_bytes(s, 32, 1024)["total"] == 3_274_698_240 + 32 * (86_507_520 + 84_480)


def test_make_weights_layout_and_determinism():
    s = O.RavenShape.tiny()
    w = O.make_weights(s, seed=0)
    names = [n for n, _ in O.state_dict_layout(s)]
    assert names[0] == "transformer.wte.weight" and names[-1] == "transformer.ln_f.weight"
    assert "transformer.prelude.0.attn.qk_bias" in names and "transformer.adapter.weight" in names
    assert w["lm_head.weight"] is w["transformer.wte.weight"]
    assert w["transformer.core_block.1.mlp.fc.weight"].shape == (2 * 704, 256)
    assert w["transformer.prelude.0.attn.qk_bias"].shape == (2, 1, 4, 64)
    w2 = O.make_weights(s, seed=0)
    assert all(torch.equal(w[k], w2[k]) for k in w)
    assert abs(w["transformer.ln_f.weight"].mean().item() - 1.0) < 0.01
    n_params = sum(math.prod(sh) for _, sh in O.state_dict_layout(O.RavenShape.nebel()))
    assert n_params == 3_564_976_800 + 0  # tied head counted once


# ----------------------------------------------------------------------------- adaptive compute
def _fake_predict(logits):
    return lambda lat: O.OracleOutput(logits=logits.unsqueeze(1), latent_states=lat)


def test_exit_entropy_closed_forms():
    V = 1000
    ev = O.ExitCriterion("entropy-diff", "auto", V)
    ev.init(torch.zeros(2, 1, 4))
    logits = torch.zeros(2, V)
    logits[1, 7] = 200.0                                   # one-hot: entropy 0; uniform: log V
    exits, out, v = ev.check(torch.zeros(2, 1, 4), _fake_predict(logits))
    assert out is not None and not exits.any()
    assert torch.allclose(ev.prev, torch.tensor([math.log(V), 0.0]), atol=2e-4)
    assert torch.allclose(v, torch.tensor([100 - math.log(V), 100.0]), atol=2e-4)   # |entropy - 100| on the first check
    exits, _, v = ev.check(torch.zeros(2, 1, 4), _fake_predict(logits))             # unchanged distribution: difference 0
    assert exits.all() and float(v.abs().max()) == 0.0
    p = torch.tensor([0.5, 0.25, 0.25])                    # entropy 1.5 ln 2
    ev3 = O.ExitCriterion("entropy-diff", 0.5, 3)
    ev3.init(torch.zeros(1, 1, 4))
    ev3.check(torch.zeros(1, 1, 4), _fake_predict(p.log().unsqueeze(0)))
    assert abs(float(ev3.prev) - 1.5 * math.log(2)) < 1e-6


def test_exit_kl_closed_forms_and_direction():
    V = 4
    ev = O.ExitCriterion("kl", "auto", V)
    ev.init(torch.zeros(1, 1, 2))
    q = torch.tensor([[0.7, 0.1, 0.1, 0.1]])
    _, _, v = ev.check(torch.zeros(1, 1, 2), _fake_predict(q.log()))
    want = sum(0.25 * (math.log(0.25) - math.log(x)) for x in q[0].tolist())       # KL(previous || current), previous uniform
    assert abs(float(v) - want) < 1e-6
    r = torch.tensor([[0.4, 0.3, 0.2, 0.1]])
    _, _, v = ev.check(torch.zeros(1, 1, 2), _fake_predict(r.log() + 3.0))         # shift invariance of log_softmax
    want = sum(a * (math.log(a) - math.log(b)) for a, b in zip(q[0].tolist(), r[0].tolist()))
    wrong = sum(b * (math.log(b) - math.log(a)) for a, b in zip(q[0].tolist(), r[0].tolist()))
    assert abs(float(v) - want) < 1e-6 and abs(want - wrong) > 1e-2                # not the reverse direction
    exits, _, v = ev.check(torch.zeros(1, 1, 2), _fake_predict(r.log()))
    assert abs(float(v)) < 1e-7 and exits.all()
    assert O.ExitCriterion("some-kl-name", "auto", V).kind == "kl" and O.ExitCriterion("minp-kl", "auto", V).kind == "minp-kl"
    with pytest.raises(ValueError):
        O.ExitCriterion("nonsense")


def test_exit_minp_kl_by_hand():
    V = 4
    ev = O.ExitCriterion("minp-kl", "auto", V)
    ev.init(torch.zeros(1, 1, 2))
    p = torch.tensor([[0.6, 0.3, 0.05, 0.05]])             # below 0.1 * 0.6: floored to 1/V, then renormalised
    _, _, v = ev.check(torch.zeros(1, 1, 2), _fake_predict(p.log()))
    filt = [0.6 / 1.4, 0.3 / 1.4, 0.25 / 1.4, 0.25 / 1.4]
    assert torch.allclose(ev.prev.exp(), torch.tensor([filt]), atol=1e-6)
    want = sum(0.25 * (math.log(0.25) - math.log(x)) for x in filt)
    assert abs(float(v) - want) < 1e-6
    assert ev.threshold == 1e-5 and O.ExitCriterion("kl", "auto", V).threshold == 1e-3


def test_exit_latent_criteria_closed_forms():
    prev = torch.tensor([[[3.0, 4.0, 0.0, 0.0], [1.0, 0.0, 0.0, 0.0]]])            # [1, 2, 4]
    ev = O.ExitCriterion("latent-diff", 0.6)
    ev.init(prev)
    _, out, v = ev.check(2 * prev, None)                   # |2x - x| / |2x| = 1/2 at both positions
    assert out is None and abs(float(v) - 0.5) < 1e-7
    cur = torch.tensor([[[6.0, 8.0, 0.0, 0.0], [2.0, 0.0, 2.0, 0.0]]])
    _, _, v = ev.check(cur, None)                          # position 0: 10/10... |cur - 2 prev| = 0 -> 0; position 1: 2 / sqrt 8
    assert abs(float(v) - (0.0 + 2 / math.sqrt(8)) / 2) < 1e-6
    ec = O.ExitCriterion("cosine", "auto")
    ec.init(prev)
    exits, _, v = ec.check(torch.tensor([[[-4.0, 3.0, 0.0, 0.0], [5.0, 0.0, 0.0, 0.0]]]), None)
    assert abs(float(v) - 0.5) < 1e-6 and not exits.any()  # orthogonal and parallel: mean cosine 1/2
    assert ec.threshold == 1e-3 and ev.threshold == 0.6 and O.ExitCriterion("latent-diff").threshold == 0.03


def test_exit_argmax_stability_and_num_steps_counting():
    ev = O.ExitCriterion("argmax-stability", 2, 5)
    ev.init(torch.zeros(1, 1, 2))
    streaks = []
    for tok in (3, 3, 1, 1, 1, 1):
        logits = torch.zeros(1, 5)
        logits[0, tok] = 1.0
        exits, _, v = ev.check(torch.zeros(1, 1, 2), _fake_predict(logits))
        streaks.append((int(v), bool(exits)))
    assert streaks == [(0, False), (1, False), (0, False), (1, False), (2, True), (3, True)]
    assert O.ExitCriterion("argmax-stability", "auto", 5).threshold == 5
    ns = O.ExitCriterion("num-steps", steps_fn=lambda i: [2, 1][i])
    ns.init(torch.zeros(3, 1, 2))
    assert not ns.check(torch.zeros(3, 1, 2), None)[0].any() and ns.check(torch.zeros(3, 1, 2), None)[0].all()
    ns.init(torch.zeros(3, 1, 2))
    assert ns.check(torch.zeros(3, 1, 2), None)[0].all()


def test_adaptive_pieces_compose_to_forward_and_greedy():
    s = O.RavenShape.tiny()
    w = O.make_weights(s, seed=0, dtype=torch.float32)
    g = torch.Generator().manual_seed(3)
    ids = torch.randint(0, s.vocab_size, (2, 6), generator=g)
    states = O.initialize_state(torch.empty(2, 6, s.n_embd), s, 1.0, g)
    want = O.forward(w, s, input_ids=ids, input_states=states, num_steps=3)
    embeds, b = O.embed_inputs(w, s, ids)
    x = states
    for _ in range(3):
        x, b = O.iterate_one_step(w, s, embeds, x, b)
    assert b == s.n_layers_in_prelude - 1 + 3 * s.n_layers_in_recurrent_block
    got = O.predict_from_latents(w, s, x)
    assert torch.equal(got.logits, want.logits)            # ln_f is applied inside predict_from_latents (RMM:886)
    sf = lambda c, sh: O.initialize_state(torch.empty(sh), s, 1.0, torch.Generator().manual_seed(50 + c))
    a = O.greedy_generate(w, s, ids, 5, state_fn=sf)
    b_ids, steps = O.generate_with_adaptive_compute(w, s, ids, 5, criterion="none", state_fn=sf)
    assert torch.equal(a, b_ids) and steps == [[s.mean_recurrence] * 2] * 5
    # a fixed schedule of recurrences per token equals forward(num_steps=k) token by token on a shared cache
    sched = [3, 1, 4, 2]
    c_ids, steps = O.generate_with_adaptive_compute(w, s, ids, 4, num_steps=4, state_fn=sf,
                                                    evaluator=O.ExitCriterion("num-steps", steps_fn=lambda i: sched[i]))
    assert steps == [[k, k] for k in sched]
    cache, cur = O.DictCache(), ids.clone()
    for call, k in enumerate(sched):
        seen = cache.get_seq_length()
        pos = torch.arange(seen, cur.shape[1])
        out = O.forward(w, s, input_ids=cur[:, pos], input_states=sf(call, (2, len(pos), s.n_embd)), num_steps=k,
                        past_key_values=cache, use_cache=True, cache_position=pos)
        cur = torch.cat([cur, out.logits[:, -1].argmax(-1, keepdim=True)], dim=-1)
    assert torch.equal(cur, c_ids)
    # token-by-token prefill with exits: same schedule, logits of each token equal the forward's
    ev = O.ExitCriterion("num-steps", steps_fn=lambda i: sched[i % 4])
    logits, _, st = O.prefill_with_varied_exit_steps(w, s, ids[:1, :4], ev, state_fn=sf)
    assert st == sched and logits.shape == (1, 4, s.vocab_size)


def test_speculative_decoding_preserves_greedy_output():
    """With deterministic (zero) initial states, drafting and verifying must reproduce plain greedy decoding, whatever
    the draft depth and the look-ahead; with the draft as deep as the verifier every drafted token is accepted."""
    s = O.RavenShape.tiny()
    w = O.make_weights(s, seed=0, dtype=torch.float32)
    ids = torch.randint(0, s.vocab_size, (1, 6), generator=torch.Generator().manual_seed(2))
    plain = O.greedy_generate(w, s, ids, 12, num_steps=4)
    for draft_steps, look in ((4, 3), (1, 3), (2, 4)):
        rec = {}
        spec = O.generate_speculative(w, s, ids, 12, draft_steps=draft_steps, lookahead_for_draft=look, num_steps=4,
                                      init_scale=0.0, record=rec)
        n = min(plain.shape[1], spec.shape[1])
        assert n >= 6 + 12 and torch.equal(plain[:, :n], spec[:, :n])
        if draft_steps == 4:
            assert all(c == [look] for c in rec["accepted"])
        assert rec["cache"].get_seq_length() == spec.shape[1] - 1       # exactly one token is still unseen by the cache
    stop = int(plain[0, 8])
    cut = O.generate_speculative(w, s, ids, 12, draft_steps=1, lookahead_for_draft=3, num_steps=4, init_scale=0.0, stop_tokens=(stop,))
    assert int(cut[0, -1]) == stop and torch.equal(cut[0], plain[0, :cut.shape[1]])


# --------------------------------------------------------------------------------------
# diffusion-style sampler
# --------------------------------------------------------------------------------------
def _diffusion_model():
    s = O.RavenShape(n_embd=64, n_heads=2, intermediate_size=96, vocab_size=128, n_layers_in_prelude=2, n_layers_in_recurrent_block=4,
                     n_layers_in_coda=2, mean_recurrence=4, block_size=64)
    w = O.make_weights(s, seed=3, dtype=torch.float32)
    ids = torch.randint(0, s.vocab_size, (1, 5), generator=torch.Generator().manual_seed(8))
    sf = lambda c, sh: O.initialize_state(torch.empty(sh), s, 1.0, torch.Generator().manual_seed(600 + c))
    return s, w, ids, sf


def test_diffusion_sampler_first_wave_position_followed_by_hand():
    """The leftmost wave position never sees the positions to its right (causal attention), and its token does not
    change while it waits, so everything the loop does to it can be restated for that position alone, each step on a
    private copy of the prompt's cache: embedding average with the previous step's, noise mixing damped by the
    recurrences it has had, `inner_recurrence` recurrences, coda and head.  Its latent state and its logits after every
    step must be the ones this hand computation gives (the token alone would not do: with random weights the argmax
    hardly moves), and the token the loop freezes at the next position their argmax.  A wrong wave offset, a cache
    rollback that drops too little or too much, a wrong damping count or mixing order, a recurrence too many or too
    few, or noise states handed out in the wrong order all change the state by far more than the tolerance (checked:
    each of these moves the top-2 logit margin in the second decimal)."""
    import copy
    s, w, ids, sf = _diffusion_model()
    n, h = ids.shape[1], s.n_embd
    num_steps, inner, a, m = 4, 2, 0.1, 0.5
    rec = {}
    got = O.generate_diffusion_style(w, s, ids, 3, num_steps=num_steps, inner_recurrence=inner, freeze_strategy="fixed", ema_embeds=a,
                                     state_noise_mixing=m, state_fn=sf, record=rec)
    # by hand
    cache0 = O.DictCache("latest-m4-compress-s4")
    out = O.forward(w, s, input_ids=ids, input_states=sf(0, (1, n, h)), num_steps=num_steps, past_key_values=cache0, use_cache=True,
                    cache_position=torch.arange(n))
    tok1 = out.logits[:, -1, :].argmax(-1, keepdim=True)
    assert int(got[0, n]) == int(tok1)
    state = sf(1, (1, 1, h))
    old_e = O.embed_inputs(w, s, torch.cat([ids, tok1], dim=1))[0][:, n:]
    pos = torch.tensor([n])
    n_hold = num_steps // inner                       # steps 0 .. n_hold freeze nothing, step n_hold + 1 freezes one position
    for t in range(n_hold + 2):
        cache = copy.deepcopy(cache0)
        e_new, block_idx = O.embed_inputs(w, s, tok1, cache=cache, cache_position=pos)
        e = e_new * (1 - a) + old_e * a
        old_e = e
        noise = sf(2 + 2 * t, (1, t + 1, h))[:, :1]   # draws: prefill, first state, then (noise, new position) per step
        mix = m / (1 + num_steps + inner * t)
        state = state * (1 - mix) + mix * noise
        for _ in range(inner):
            state, block_idx = O.iterate_one_step(w, s, e, state, block_idx, cache=cache, cache_position=pos)
        logits = O.predict_from_latents(w, s, state, cache=cache, cache_position=pos).logits[0, 0]
        assert rec["log"][t]["cache_index"] == n and rec["log"][t]["wave"] == t + 1
        assert torch.allclose(rec["log"][t]["first_state"], state[0, 0], rtol=1e-4, atol=1e-5), t
        assert torch.allclose(rec["log"][t]["first_logits"], logits, rtol=1e-4, atol=1e-5), t
    assert int(got[0, n + 1]) == int(logits.argmax())
    assert rec["log"][n_hold + 2]["cache_index"] == n + 1      # the position is frozen: the next wave starts behind it
    assert rec["draws"] == 2 + 2 * rec["diffusion_steps"]


def test_diffusion_sampler_fixed_schedule_closed_form():
    """freeze_strategy "fixed", headway 1: nothing freezes during steps 0 .. num_steps // inner, then one position per
    step; the wave grows to num_steps // inner + 2 positions and stays there.  Counters follow in closed form."""
    s, w, ids, sf = _diffusion_model()
    n, num_steps, inner, max_new = ids.shape[1], 4, 2, 5
    rec = {}
    out = O.generate_diffusion_style(w, s, ids, max_new, num_steps=num_steps, inner_recurrence=inner, freeze_strategy="fixed",
                                     state_fn=sf, record=rec)
    hold = num_steps // inner                         # 2
    steps = hold + 1 + (max_new - 1)                  # the prefill froze one token already
    waves = [min(t + 1, hold + 2) for t in range(steps)]
    assert out.shape == (1, n + max_new) and torch.equal(out[:, :n], ids)
    assert rec["diffusion_steps"] == steps and rec["num_standing_waves"] == 0
    assert rec["num_core_forward_passes"] == 1 + inner * steps
    assert rec["num_tokens_forward"] == n + inner * sum(waves)
    assert rec["num_cache_clears"] == sum(wv if t <= hold else wv - 1 for t, wv in enumerate(waves))
    per_pos = [num_steps] * n + [num_steps + inner * (hold + 2)] + [inner * (hold + 2)] * (max_new - 2) + [inner * (hold + 1)]
    assert rec["recurrence_per_position"].tolist() == [per_pos]
    assert rec["cache"].get_seq_length() == n + max_new - 1      # every frozen position but the newest is cached
    # the cache holds, for the frozen positions, one entry per prelude / core slot / coda block
    assert sorted(rec["cache"].key_cache.keys()) == [-2, -1, 0, 1, 2, 3, 4, 5]
    assert all(sorted(c.keys()) == list(range(n + max_new - 1)) for c in rec["cache"].key_cache.values())


def test_diffusion_sampler_never_freezing_and_standing_waves():
    """exit_t = 0 never freezes a position: the wave grows by `headway` per step up to max_wavefront and then stands;
    the loop ends at max_diffusion_steps with the prompt and the prefill's token only, and an empty wave in the cache."""
    s, w, ids, sf = _diffusion_model()
    n = ids.shape[1]
    rec = {}
    out = O.generate_diffusion_style(w, s, ids, 4, num_steps=4, inner_recurrence=1, freeze_strategy="latent-diff", exit_t=0.0,
                                     max_wavefront=3, max_diffusion_steps=5, state_fn=sf, record=rec)
    assert out.shape == (1, n + 1)
    assert rec["diffusion_steps"] == 6                          # leaves in the step after the limit, before counting it
    assert [e["wave"] for e in rec["log"]] == [1, 2, 3, 3, 3, 3, 3]
    assert rec["num_standing_waves"] == 5
    assert rec["cache"].get_seq_length() == n
    assert rec["num_cache_clears"] == 1 + 2 + 3 * 5
    # a huge threshold freezes every position that has a previous state to compare with; the prefill's token stays
    rec2 = {}
    out2 = O.generate_diffusion_style(w, s, ids, 4, num_steps=4, inner_recurrence=1, freeze_strategy="latent-diff", exit_t=1e9,
                                      state_fn=sf, record=rec2)
    assert out2.shape == (1, n + 4) and int(out2[0, n]) == int(out[0, n])
    assert all(e["frozen"] >= b["frozen"] for b, e in zip(rec2["log"], rec2["log"][1:]))


# ----------------------------------------------------------------------------- test-time noise
class _Draws:
    """Deterministic stand-ins for randn_like / rand(1)."""

    def __init__(self, normal=None, uniform=0.25, seed=None):
        self._n, self._u = normal, uniform
        self._g = None if seed is None else torch.Generator().manual_seed(seed)

    def normal(self, x):
        if self._g is not None:
            return torch.randn(x.shape, generator=self._g).to(x.dtype)
        return torch.full_like(x, self._n)

    def uniform(self, x):
        return torch.tensor([self._u], dtype=x.dtype)


def _noisy(kind, t=0.3):
    import dataclasses
    s = dataclasses.replace(O.RavenShape.tiny(), test_time_noise=t, test_time_noise_type=kind)
    return s, O.make_weights(s, seed=0, dtype=torch.float32)


def test_noise_amplitude_and_per_type_coefficients_closed_form():
    """x = 0, noise = 1, no renormalisation: the output is the coefficient c itself.  n = t * std * sqrt(h) with
    std = sqrt(2/(5h)) is t * sqrt(2/5) whatever the width (RMM:817, raven_config_minimal.py:86)."""
    t = 0.3
    n = t * math.sqrt(0.4)
    want = {("fixed", 0): n, ("fixed", 5): n, ("geom", 0): n, ("geom", 2): n / 3, ("sqrt", 0): n, ("sqrt", 3): n / 2,
            ("line", 0): 1.0, ("line", 1): 0.75, ("line", 3): max(n, 0.25), ("chi", 0): 2 * 0.25 * n}
    for (kind, k), c in want.items():
        s, w = _noisy(kind, t)
        x = torch.zeros(1, 2, s.n_embd)
        y = O.inject_noise(x, k, w, s, _Draws(normal=1.0), renorm=False)
        assert torch.allclose(y, torch.full_like(y, c), rtol=1e-6, atol=0), (kind, k)
        # and the state keeps 1 - c: x = 1, noise = 0
        y = O.inject_noise(torch.ones(1, 2, s.n_embd), k, w, s, _Draws(normal=0.0), renorm=False)
        assert torch.allclose(y, torch.full_like(y, 1 - c), rtol=1e-6, atol=1e-7), (kind, k)


def test_noise_off_is_identity_and_zero_noise_leaves_the_norm():
    s, w = _noisy("fixed", 0.0)
    x = torch.randn(2, 3, s.n_embd)
    assert O.inject_noise(x, 1, w, s, _Draws(normal=1.0)) is x
    # RMSNorm does not see a scale: x * (1 - n) + 0 renormalises to norm_4(x)
    s, w = _noisy("fixed", 0.3)
    got = O.inject_noise(x, 1, w, s, _Draws(normal=0.0))
    want = O.rmsnorm(x, w[f"transformer.core_block.{s.n_layers_in_recurrent_block - 1}.norm_4.weight"], s.norm_eps)
    assert torch.allclose(got, want, rtol=1e-5, atol=1e-6)


def test_line_noise_replaces_the_state_at_step_zero_inside_forward():
    """With "line" the first recurrence sees pure noise (c = 1 at step 0): the forward pass no longer depends on
    input_states, which also fixes WHERE the injection sits (in front of the adapter) and that steps count from 0."""
    s, w = _noisy("line", 0.3)
    g = torch.Generator().manual_seed(5)
    ids = torch.randint(0, s.vocab_size, (1, 6), generator=g)
    a = torch.randn(1, 6, s.n_embd, generator=g)
    b = torch.randn(1, 6, s.n_embd, generator=g)
    out_a = O.forward(w, s, input_ids=ids, input_states=a, noise_draws=_Draws(seed=9))
    out_b = O.forward(w, s, input_ids=ids, input_states=b, noise_draws=_Draws(seed=9))
    assert torch.equal(out_a.logits, out_b.logits)
    other = O.forward(w, s, input_ids=ids, input_states=a, noise_draws=_Draws(seed=10))
    assert not torch.equal(out_a.logits, other.logits)
    # "fixed" keeps 1 - n of the state: there the two do differ
    s2, _ = _noisy("fixed", 0.3)
    out_c = O.forward(w, s2, input_ids=ids, input_states=a, noise_draws=_Draws(seed=9))
    out_d = O.forward(w, s2, input_ids=ids, input_states=b, noise_draws=_Draws(seed=9))
    assert not torch.equal(out_c.logits, out_d.logits)


def test_bench_counts_the_same_bytes_and_keeps_the_oracle_to_its_cpu_leg(pkg):
    """bench.py carries its own statement of an iteration's algorithmic bytes (the product side may not import the
    oracle); it must agree with the pinned count above, and the oracle import must sit inside cpu_baseline only."""
    import ast
    import os
    import bench
    s = O.RavenShape.nebel()
    cfg = pkg.RavenConfig()
    for B, T in ((1, 1024), (8, 640), (32, 1024)):
        mine, pinned = bench.core_iteration_bytes(cfg, B, T), O.core_iteration_bytes(s, B, T)
        assert {k: mine[k] for k in pinned} == pinned
        # the schedule of a call with several recurrences: the embedding half of the adapter (5280 x 5280 bf16) leaves the
        # per-iteration count, its fp32 sums (B x 5280) enter it; that half and the sums are counted once per call
        split = bench.core_iteration_bytes(cfg, B, T, adapter_split=True)
        assert split["total"] == pinned["total"] - 5280 * 5280 * 2 + B * 5280 * 4
        assert bench.adapter_once_bytes(cfg, B) == 5280 * 5280 * 2 + B * 5280 * 4
    tree = ast.parse(open(os.path.join(os.path.dirname(bench.__file__), "bench.py")).read())
    holders = [fn.name for fn in ast.walk(tree) if isinstance(fn, ast.FunctionDef)
               for node in ast.walk(fn) if isinstance(node, (ast.Import, ast.ImportFrom))
               and "oracle" in (getattr(node, "module", None) or " ".join(a.name for a in node.names))]
    top = [node for node in tree.body if isinstance(node, (ast.Import, ast.ImportFrom))
           and "oracle" in (getattr(node, "module", None) or " ".join(a.name for a in node.names))]
    assert holders == ["cpu_baseline"] and not top


# ----------------------------------------------------------------------------- diffusion sampler, every wave position
class _RowContext:
    """What one position sees, kept position by position instead of in a step-indexed cache: `done[q][step_idx]` holds the
    key/value row that position q wrote at block `step_idx` the last time it was computed.  The position being computed
    reads, at block `step_idx`, the rows of all positions to its left -- from the same block of the same recurrence when
    that position was computed earlier in this pass (it is part of the same wave), else from that position's last pass:
    its last recurrence for a core block (which is what a cache that keeps one slot per core block holds)."""

    def __init__(self, shape):
        self.s = shape
        self.done = {}      # position -> {step_idx: (k, v)} of its last complete pass
        self.pass_rows = {}  # position -> {step_idx: (k, v)} of the pass in progress (all positions of the current wave)
        self.pos = None
        self.write = True

    def core_class(self, step_idx):
        n_pre, n_core = self.s.n_layers_in_prelude, self.s.n_layers_in_recurrent_block
        return None if step_idx < n_pre else (step_idx - n_pre) % n_core   # coda blocks (negative) never get here

    def rows_of(self, q, step_idx):
        if q in self.pass_rows and step_idx in self.pass_rows[q]:
            return self.pass_rows[q][step_idx]
        rows = self.done[q]                       # a position from an earlier pass
        cls = self.core_class(step_idx)
        if step_idx < 0 or cls is None:           # prelude and coda blocks run once per pass
            return rows[step_idx]
        last = max(i for i in rows if i >= self.s.n_layers_in_prelude and self.core_class(i) == cls)
        return rows[last]                         # its last recurrence of that core block

    def update(self, k, v, step_idx, lookup_strategy=None):
        left = [self.rows_of(q, step_idx) for q in range(self.pos)]
        if self.write:
            self.pass_rows.setdefault(self.pos, {})[step_idx] = (k, v)
        ks = torch.cat([r[0] for r in left] + [k], dim=2)
        vs = torch.cat([r[1] for r in left] + [v], dim=2)
        return ks, vs

    def end_pass(self):
        self.done.update(self.pass_rows)
        self.pass_rows = {}


def _one_position(s, w, ctx, p, token, state, n_rec, embed_mix=None, write=True):
    """Prelude, n_rec recurrences and coda for position p alone; returns (embedding used, state, logits)."""
    ctx.pos, ctx.write = p, write
    cp = torch.tensor([p])
    e, block_idx = O.embed_inputs(w, s, token.view(1, 1), cache=ctx, cache_position=cp)
    if embed_mix is not None:
        e = embed_mix(e)
    for _ in range(n_rec):
        state, block_idx = O.iterate_one_step(w, s, e, state, block_idx, cache=ctx, cache_position=cp)
    logits = O.predict_from_latents(w, s, state, cache=ctx, cache_position=cp).logits[0, 0] if n_rec else None
    return e, state, logits


@pytest.mark.parametrize("strategy,exit_t", [("fixed", None), ("latent-diff", 0.35), ("latent-diff", 0.2)])
def test_diffusion_sampler_every_wave_position_followed_position_by_position(strategy, exit_t):
    """The sampler advances a wave of positions together, over a cache with one slot per core block whose wave part is
    rolled back after every step.  Here the same text is produced one position at a time, with no step-indexed cache,
    no roll-back and no batching: every position keeps the key/value rows of its own last computation, and a position
    reads its left neighbours row by row (_RowContext).  The bookkeeping is restated per position as well: a position's
    token is the frozen one or the previous step's prediction of its left neighbour; its embedding is averaged with its
    own previous one; its state is mixed with noise damped by its own recurrence count; "fixed" freezes the leftmost
    wave position from step num_steps // inner + 1 on, "latent-diff" everything up to the rightmost position whose state
    moved by less than exit_t since the previous step.  States and logits of EVERY wave position must agree after every
    step, and the frozen text at the end -- so a wrong wave offset, roll-back count, slot, guess alignment or damping
    count for any position, not only the leftmost, shows."""
    s, w, ids, sf = _diffusion_model()
    n, h = ids.shape[1], s.n_embd
    num_steps, inner, a, m, max_new = 4, 2, 0.1, 0.5, 5
    rec = {}
    kw = dict(freeze_strategy=strategy) if exit_t is None else dict(freeze_strategy=strategy, exit_t=exit_t)
    got = O.generate_diffusion_style(w, s, ids, max_new, num_steps=num_steps, inner_recurrence=inner, ema_embeds=a, state_noise_mixing=m,
                                     state_fn=sf, record=rec, **kw)
    # ---- position by position
    ctx = _RowContext(s)
    x0 = sf(0, (1, n, h))
    for p in range(n):                                             # the prompt, num_steps recurrences per position
        _, _, logits = _one_position(s, w, ctx, p, ids[0, p], x0[:, p:p + 1], num_steps)
    ctx.end_pass()
    text = ids[0].tolist() + [int(logits.argmax())]                # frozen tokens
    n_frozen = n + 1
    guess = {}                                                     # position -> predicted token, for positions not frozen yet
    state = {n: sf(1, (1, 1, h))}
    count = {n: num_steps}                                         # recurrences a position has had (the prefill counts for n)
    old_e = {n: _one_position(s, w, ctx, n, torch.tensor(text[n]), None, 0, write=False)[0]}
    prev_state = None
    hold = num_steps // inner
    draws, t = 2, 0
    while n_frozen - n < max_new:
        first = n_frozen - 1                                       # the newest frozen token is the wave's leftmost position
        wave = sorted(state)
        assert wave == list(range(first, first + len(wave)))
        entry = rec["log"][t]
        assert (entry["cache_index"], entry["wave"]) == (first, len(wave)), t
        noise = sf(draws, (1, len(wave), h))
        after, logit_of = {}, {}
        for i, p in enumerate(wave):
            tok = text[p] if p < n_frozen else guess[p]
            x = state[p]
            mix = m / (1 + count.get(p, 0))
            x = x * (1 - mix) + mix * noise[:, i:i + 1]
            carry = old_e.get(p)
            e, x, lg = _one_position(s, w, ctx, p, torch.tensor(tok), x, inner,
                                     embed_mix=lambda new, c=carry: new * (1 - a) + (c * a if c is not None else 0))
            old_e[p], after[p], logit_of[p] = e, x, lg
            count[p] = count.get(p, 0) + inner
            assert torch.allclose(entry["wave_states"][i], x[0, 0], rtol=1e-4, atol=1e-5), (t, p)
            assert torch.allclose(entry["wave_logits"][i], lg, rtol=1e-4, atol=1e-5), (t, p)
        ctx.end_pass()
        for p in wave:                                             # predictions for the positions behind the frozen text
            if p + 1 >= n_frozen:
                guess[p + 1] = int(logit_of[p].argmax())
        new_pos = wave[-1] + 1
        after[new_pos] = sf(draws + 1, (1, 1, h)).to(torch.bfloat16).to(x0.dtype)
        draws += 2
        if strategy == "fixed":
            new_frozen = n_frozen + (1 if t > hold else 0)
        else:
            new_frozen = n_frozen
            if prev_state is not None:
                moved = {p: float((after[p] - prev_state[p]).norm() / after[p].norm()) for p in after if p in prev_state}
                settled = [p for p, v in moved.items() if v < exit_t]
                if settled:
                    new_frozen = max(settled) + 1
        for p in range(n_frozen, new_frozen):
            text.append(guess[p])
        n_frozen = new_frozen
        state = {p: x for p, x in after.items() if p >= n_frozen - 1}
        old_e = {p: e for p, e in old_e.items() if p >= n_frozen - 1}
        prev_state = dict(state)
        assert entry["frozen"] == n_frozen, t
        t += 1
    assert got[0].tolist() == text[:got.shape[1]] and got.shape[1] == n_frozen
    assert t == rec["diffusion_steps"]


def test_repetition_penalty_by_hand_and_against_the_library_processor():
    """RMM:2047-2061 is the rule of transformers' RepetitionPenaltyLogitsProcessor: seen tokens' logits are divided by the
    penalty when positive and multiplied when negative; a token seen twice is penalised once; unseen tokens stay."""
    from transformers import RepetitionPenaltyLogitsProcessor
    logits = torch.tensor([[2.0, -3.0, 0.5, 4.0], [1.0, 1.0, -1.0, 0.0]])
    ids = torch.tensor([[0, 1, 1], [2, 2, 3]])
    got = O.repetition_penalty(logits, ids, 2.0)
    assert got.tolist() == [[1.0, -6.0, 0.5, 4.0], [1.0, 1.0, -2.0, 0.0]]
    g = torch.Generator().manual_seed(5)
    big, seq = torch.randn(3, 50, generator=g), torch.randint(0, 50, (3, 12), generator=g)
    assert torch.equal(O.repetition_penalty(big, seq, 1.3), RepetitionPenaltyLogitsProcessor(1.3)(seq, big.clone()))
    # greedy_generate with a penalty = the plain loop with the library's processor applied to the growing sequence
    s = O.RavenShape.tiny()
    w = O.make_weights(s, seed=0, dtype=torch.float32)
    proc = RepetitionPenaltyLogitsProcessor(1.6)
    changed = 0
    for seed in range(1000, 1012):
        prompt = torch.randint(0, s.vocab_size, (1, 6), generator=torch.Generator().manual_seed(seed))
        seq, cache = prompt.clone(), O.DictCache()
        for _ in range(14):
            pos = torch.arange(cache.get_seq_length(), seq.shape[1])
            out = O.forward(w, s, input_ids=seq[:, pos], past_key_values=cache, use_cache=True, cache_position=pos, init_scale=0.0)
            seq = torch.cat([seq, proc(seq, out.logits[:, -1].float().clone()).argmax(-1, keepdim=True)], dim=-1)
        assert torch.equal(O.greedy_generate(w, s, prompt, 14, penalty=1.6), seq), seed
        changed += not torch.equal(O.greedy_generate(w, s, prompt, 14), seq)
    assert changed >= 1                                                   # some of these streams repeat without the penalty
