"""Full-size checks at the 3.5b shape (bf16, 512-token prompts, 32 recurrences, up to 32 sequences), where the CPU
oracle would take minutes per call: properties that hold independently of the size and need no reference values, and
one whole forward in fp32 against the fp32 oracle (short prompt, two recurrences), which pins the indexing of every
part of the model at its real strides.

  * determinism: the same call twice gives the same bits; a HIP-graph replay gives the bits of the eager launches;
  * permutation equivariance: shuffling the sequences of a batch shuffles logits, latents and cache rows, bit for bit
    (every row's arithmetic is its own; this is a test of batch / head / position indexing at the real strides);
  * capacity independence: a cache with room for more positions gives the same bits;
  * the cache accounting of the reference's notebooks at this size.

Comparisons between DIFFERENT kernel paths (a sequence alone against the same sequence in a batch, cache-then-decode
against one uncached forward) are not asserted at this size: with random N(0, 0.02) weights the recurrent block
amplifies bf16 rounding so strongly that the CPU oracle in bf16 is itself 0.39 (rel-L2) away from its fp32 run after
one recurrence and uncorrelated after four, and so is every other bf16 implementation, this one included (measured:
0.385 / 0.382 / 0.385 for the three paths of this package against the same fp32 run).  Those comparisons are made
per kernel and per block in test_gpu_kernels.py / test_gpu_model.py, where they are meaningful."""

import pytest
import torch

pytestmark = pytest.mark.gpu

PROMPT, R = 512, 32


@pytest.fixture(autouse=True)
def _release_device_memory():
    """The caches of these tests are tens of GB each: give them back before the next test allocates its own."""
    yield
    import gc
    gc.collect()
    torch.cuda.empty_cache()


@pytest.fixture(scope="module")
def nebel(pkg):
    model = pkg.RavenForCausalLM(pkg.RavenConfig(), device="cuda:0", dtype=torch.bfloat16)
    torch.manual_seed(0)
    with torch.no_grad():
        for name, p in model.state_dict().items():
            if name == "freqs_cis" or name == "lm_head.weight":
                continue
            p.normal_(1.0 if p.dim() == 1 else 0.0, 0.02)
    return model


def _prompt(B, n=PROMPT, seed=1):
    return torch.randint(0, 65536, (B, n), generator=torch.Generator().manual_seed(seed)).cuda()


@pytest.mark.parametrize("B", [1, 8, 32])
def test_decode_is_deterministic_and_graph_replay_equals_eager(pkg, nebel, B):
    """1, 8 and 32 sequences, 512-token prompt: four decode steps from the same prefilled cache, three times (eager
    launches, a captured HIP graph, a second captured graph): the same bits every time.  One sequence takes the one-row
    schedule (every norm in a GEMV prologue, all 32 recurrences in one raven_core_iterations call with the adapter split
    by columns), 8 and 32 the multi-row one."""
    ids = _prompt(B)
    cache = pkg.HuginnDynamicCache(max_length=PROMPT + 8)
    h = nebel.config.n_embd
    out = nebel(input_ids=ids, input_states=torch.zeros(B, PROMPT, h, device="cuda", dtype=torch.bfloat16), past_key_values=cache,
                use_cache=True, cache_position=torch.arange(PROMPT).cuda(), num_steps=R)
    first = out.logits[:, -1].argmax(-1)
    k0, v0 = cache._k.clone(), cache._v.clone()
    runs = []
    for use_graph in (False, True, True):
        cache._k.copy_(k0)
        cache._v.copy_(v0)
        cache.clear_last_k_entries(cache.get_seq_length() - PROMPT)
        runner = pkg.DecodeRunner(nebel, cache, B, R, greedy=True, use_graph=use_graph)
        tok, rec = first, []
        for _ in range(4):
            logits, nxt, latents = runner.step(tok, torch.zeros(B, h, device="cuda", dtype=torch.bfloat16))
            rec.append((logits.clone(), nxt.clone(), latents.clone()))
            tok = nxt.clone()
        runs.append(rec)
    for other in runs[1:]:
        for a, b in zip(runs[0], other):
            assert all(torch.equal(x, y) for x, y in zip(a, b))
    b2 = min(B, 2)
    again = [nebel(input_ids=ids[:b2, :48].contiguous(), input_states=torch.zeros(b2, 48, h, device="cuda", dtype=torch.bfloat16),
                   num_steps=R).logits for _ in range(2)]
    assert torch.equal(again[0], again[1])


@pytest.mark.parametrize("B", [1, 8, 32])
def test_full_token_decode_256_greedy_tokens(pkg, nebel, B):
    """The full-token decode configuration at 1, 8 and 32 sequences: 512-token random prompt, 256 greedy tokens at r = 32
    (prefill through forward(), then one HIP-graph replay per token).  Zero initial states make the run reproducible:
    the graph run and the eager run produce the same 256 tokens; all ids are inside the vocabulary; the cache holds
    512 + 255 positions in all 132 step entries."""
    ids = _prompt(B, seed=10 + B)
    gc = pkg.GenerationSettings(max_new_tokens=256)
    runs = []
    for use_graph in (True, False):
        out = nebel.generate_minimal(ids, gc, num_steps=R, init_scale=0.0, stop_tokens=set(), use_graph=use_graph)
        assert out.shape == (B, PROMPT + 256)
        assert torch.equal(out[:, :PROMPT], ids)
        new = out[:, PROMPT:]
        assert int(new.min()) >= 0 and int(new.max()) < 65536
        runs.append(new.clone())
    assert torch.equal(runs[0], runs[1]), "graph replay and eager launches must pick the same tokens"
    # three tokens on a cache of the same capacity (how many workgroups split a sequence's positions follows from the
    # capacity, and with it the order of the fp32 additions): the same first tokens
    gc2 = pkg.GenerationSettings(max_new_tokens=3, return_dict_in_generate=True)
    res = nebel.generate_minimal(ids, gc2, num_steps=R, init_scale=0.0, stop_tokens=set(),
                                 past_key_values=pkg.HuginnDynamicCache(max_length=PROMPT + 256))
    assert torch.equal(res.sequences[:, PROMPT:], runs[0][:, :3])
    assert res.past_key_values.get_seq_length() == PROMPT + 2
    for step in (0, 1, 2, 129, -1, -2):  # first and last of the 132 step entries hold every position
        assert res.past_key_values.key_cache[step][PROMPT + 1].shape == (B, 55, 96)


def _prefill_and_two_steps(pkg, model, ids, states, max_length):
    n = ids.shape[1]
    cache = pkg.HuginnDynamicCache(max_length=max_length)
    out = model(input_ids=ids, input_states=states[:, :n].contiguous(), past_key_values=cache, use_cache=True,
                cache_position=torch.arange(n).cuda(), num_steps=R)
    outs, nxt = [out], out.logits[:, -1].argmax(-1, keepdim=True)
    for i in range(2):
        step = model(input_ids=nxt, input_states=states[:, n + i:n + i + 1].contiguous(), past_key_values=cache,
                     use_cache=True, cache_position=torch.tensor([n + i]).cuda(), num_steps=R)
        outs.append(step)
        nxt = step.logits[:, -1].argmax(-1, keepdim=True)
    return outs, cache


def test_batch_permutation_and_cache_capacity_leave_every_bit_in_place(pkg, nebel):
    """Every product's accumulation order is the same for every tile position in this library's kernels, so a permutation of
    the sequences permutes the results bit for bit."""
    B, n = 32, 128
    ids = _prompt(B, n, seed=2)
    g = torch.Generator(device="cuda").manual_seed(3)
    states = (torch.randn(B, n + 2, nebel.config.n_embd, device="cuda", generator=g) * 0.632).to(torch.bfloat16)
    base, cache = _prefill_and_two_steps(pkg, nebel, ids, states, n + 2)
    perm = torch.randperm(B, generator=torch.Generator().manual_seed(4)).cuda()
    shuffled, cache_p = _prefill_and_two_steps(pkg, nebel, ids[perm].contiguous(), states[perm].contiguous(), n + 2)
    roomy, cache_r = _prefill_and_two_steps(pkg, nebel, ids, states, 2 * n + 77)
    for a, b, c in zip(base, shuffled, roomy):
        assert torch.equal(a.logits[perm], b.logits) and torch.equal(a.latent_states[perm], b.latent_states)
        assert torch.equal(a.logits, c.logits)
    for step in (0, 1, 2, 3, 64, 129, -1, -2):
        for pos in (0, 63, n - 1, n, n + 1):
            assert torch.equal(cache.key_cache[step][pos][perm], cache_p.key_cache[step][pos]), (step, pos)
            assert torch.equal(cache.value_cache[step][pos], cache_r.value_cache[step][pos]), (step, pos)
    assert cache.get_seq_length() == n + 2
    # cache size accounting at full size: 132 step entries x positions x batch x 55 x 96 x 2 bytes, key bytes doubled
    assert cache.get_memory_usage() == 132 * (n + 2) * B * 55 * 96 * 2 * 2 / 2 ** 20


def test_fp32_model_at_the_3_5b_shape_cache_equivalence(pkg):
    """The whole path in fp32 at h = 5280, hd = 96, I = 17920 (what the reference can run too): prompt through the cache
    and one decode step against one forward without a cache, the reference's own check of its cache
    (checkpoint_to_hf_converter.py:151-166).  Two recurrences keep the comparison meaningful: rounding differences
    grow by about an order of magnitude per recurrence with random weights."""
    model = pkg.RavenForCausalLM(pkg.RavenConfig(), device="cuda:0", dtype=torch.float32)
    torch.manual_seed(0)
    with torch.no_grad():
        for name, p in model.state_dict().items():
            if name == "freqs_cis" or name == "lm_head.weight":
                continue
            p.normal_(1.0 if p.dim() == 1 else 0.0, 0.02)
    B, n, h = 2, 8, model.config.n_embd
    ids = _prompt(B, n + 1, seed=5)
    g = torch.Generator(device="cuda").manual_seed(6)
    states = torch.randn(B, n + 1, h, device="cuda", generator=g) * 0.632
    full = model(input_ids=ids, input_states=states, num_steps=2)
    cache = pkg.HuginnDynamicCache()
    model(input_ids=ids[:, :n].contiguous(), input_states=states[:, :n].contiguous(), past_key_values=cache, use_cache=True,
          cache_position=torch.arange(n).cuda(), num_steps=2)
    step = model(input_ids=ids[:, n:].contiguous(), input_states=states[:, n:].contiguous(), past_key_values=cache, use_cache=True,
                 cache_position=torch.tensor([n]).cuda(), num_steps=2)
    a, b = step.latent_states[:, -1].float(), full.latent_states[:, -1].float()
    assert torch.isfinite(step.logits).all() and ((a - b).norm() / b.norm()).item() <= 1e-3
    assert step.logits.shape == (B, 1, 65536) and cache.get_seq_length() == n + 1
    out = model.generate_minimal(ids[:1, :n].contiguous(), pkg.GenerationSettings(max_new_tokens=3), num_steps=2, init_scale=0.0,
                                 stop_tokens=set())
    assert out.shape == (1, n + 3)


def test_fp32_whole_forward_at_the_3_5b_shape_against_the_fp32_oracle(pkg):
    """Embedding (65536 x 5280, scaled), two prelude blocks, two recurrences of adapter + four core blocks, two coda
    blocks, ln_f on the latents and again on the coda output, tied LM head: an 8-token prompt through the cache and one
    decode step, in fp32 against the fp32 oracle (RMM:638-724) -- logits, latent states, and the key / value rows of the
    step entries 0, 1 (prelude), 2 and 9 (first and last core step), -1 and -2 (coda).  In fp32 a wrong slot, stride,
    head or column shows as an O(1) difference, while rounding differences stay small: per kernel they are 1e-6, and the
    recurrent block amplifies them by about an order of magnitude per recurrence with random weights, hence the bars
    below for what sits behind two recurrences (the first block's rows are held to the per-kernel fp32 bar)."""
    from oracle import raven_oracle as O
    from test_gpu_kernels import check, close
    s = O.RavenShape.nebel()
    model = pkg.RavenForCausalLM(pkg.RavenConfig(), device="cuda:0", dtype=torch.float32)
    torch.manual_seed(0)
    with torch.no_grad():
        for name, p in model.state_dict().items():
            if name == "freqs_cis" or name == "lm_head.weight":
                continue
            p.normal_(1.0 if p.dim() == 1 else 0.0, 0.02)
    w = {k: v.detach().cpu() for k, v in model.state_dict().items() if k != "freqs_cis"}
    w["lm_head.weight"] = w["transformer.wte.weight"]
    w["freqs_cis"] = O.rope_table(s.head_dim, s.block_size, s.rope_base)
    B, n, h, r = 2, 8, s.n_embd, 2
    g = torch.Generator().manual_seed(5)
    ids = torch.randint(0, s.vocab_size, (B, n + 1), generator=g)
    ids[0, 0], ids[1, 0], ids[0, n] = 0, s.vocab_size - 1, s.vocab_size - 1   # first and last row of the embedding table
    states = O.initialize_state(torch.empty(B, n + 1, h), s, 1.0, g)
    ref_cache, cache = O.DictCache(), pkg.HuginnDynamicCache()
    steps = [(ids[:, :n], states[:, :n], torch.arange(n)), (ids[:, n:], states[:, n:], torch.tensor([n]))]
    for i, (tok, st, cp) in enumerate(steps):
        want = O.forward(w, s, input_ids=tok, input_states=st, past_key_values=ref_cache, use_cache=True, cache_position=cp, num_steps=r)
        got = model(input_ids=tok.cuda(), input_states=st.cuda(), past_key_values=cache, use_cache=True, cache_position=cp.cuda(),
                    num_steps=r)
        e_lat, e_log = close(got.latent_states, want.latent_states, "latents"), close(got.logits, want.logits, "logits")
        print(f"fp32 whole forward at the 3.5b shape, call {i}: latents max-abs {e_lat[0]:.3e} rel-L2 {e_lat[1]:.3e}; "
              f"logits max-abs {e_log[0]:.3e} rel-L2 {e_log[1]:.3e} (|logit|max {want.logits.abs().max():.2f})")
        assert got.logits.shape == (B, tok.shape[1], 65536) and got.logits.dtype == torch.float32
        assert e_lat[1] <= 5e-4 and e_log[1] <= 5e-4, (e_lat, e_log)   # seen: 9e-5 and 1.5e-4
        assert torch.equal(got.logits[:, -1].argmax(-1).cpu(), want.logits[:, -1].argmax(-1))
    assert cache.get_seq_length() == ref_cache.get_seq_length() == n + 1
    assert sorted(cache.key_cache.keys()) == sorted(ref_cache.key_cache.keys()) == [-2, -1] + list(range(10))
    for step in (0, 1, 2, 9, -1, -2):
        for pos in (0, n - 1, n):
            ek = close(cache.key_cache[step][pos], ref_cache.key_cache[step][pos], f"K[{step}][{pos}]")
            ev = close(cache.value_cache[step][pos], ref_cache.value_cache[step][pos], f"V[{step}][{pos}]")
            print(f"  step {step:2d} pos {pos}: K rel-L2 {ek[1]:.3e}  V rel-L2 {ev[1]:.3e}")
            if step in (0, 1, 2):   # in front of the recurrence's amplification: the per-kernel fp32 bar (seen: 3e-7 .. 4e-6)
                check(cache.key_cache[step][pos], ref_cache.key_cache[step][pos], torch.float32, f"K[{step}][{pos}]")
                check(cache.value_cache[step][pos], ref_cache.value_cache[step][pos], torch.float32, f"V[{step}][{pos}]")
            assert ek[1] <= 5e-4 and ev[1] <= 5e-4, (step, pos, ek, ev)   # seen behind two recurrences: 1e-5 .. 1.2e-4
