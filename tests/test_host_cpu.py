"""CPU-side checks: the C-ABI library loads and exports every symbol the header declares, and the
host logic (config, cache bookkeeping, step remaps) agrees with the oracle's brute-force model.
No kernel is launched here."""

import ctypes
import os
import re

import pytest
import torch

from oracle import raven_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "raven_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(raven_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(pkg):
    assert os.path.exists(pkg.hip.LIB_PATH), "libraven_hip.so has not been built"
    lib = ctypes.CDLL(pkg.hip.LIB_PATH)
    names = _declared_functions()
    assert len(names) >= 16
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in raven_hip.h but not exported"
    assert sorted(pkg.hip.SIGNATURES) == names, "the ctypes table and the header disagree"


def test_library_identity_and_argument_errors(pkg):
    lib = pkg.hip.load()
    assert lib.raven_version() >= 1 and lib.raven_arch() == b"gfx950"
    # argument validation happens before any launch, so it can be exercised without a GPU
    rc = lib.raven_rmsnorm_residual(None, None, None, None, None, None, None, 1, 5280, 1e-6, 1, None)
    assert rc < 0 and b"null" in lib.raven_last_error()
    rc = lib.raven_gemm(1, 1, None, 1, 1, 16, 7, 1, 0, None)
    assert rc < 0 and b"multiple" in lib.raven_last_error()
    rc = lib.raven_rmsnorm_residual(1, None, 1, 1, None, None, None, 1, 5280, 1e-6, 7, None)
    assert rc < 0 and b"dtype" in lib.raven_last_error()
    dims = pkg.hip.make_dims(5280, 55, 17920, 1e-6, torch.bfloat16)
    n1 = lib.raven_block_workspace_bytes(ctypes.byref(dims), 1)
    n32 = lib.raven_block_workspace_bytes(ctypes.byref(dims), 32)
    assert 0 < n1 < n32 and n1 % 256 == 0


def test_wrappers_refuse_cpu_tensors(pkg):
    x = torch.zeros(1, 16)
    with pytest.raises(pkg.hip.RavenHipError, match="GPU"):
        pkg.hip.rmsnorm_residual(x, torch.ones(16), 1e-6)


def test_config_matches_reference_defaults_and_oracle(pkg):
    cfg = pkg.RavenConfig()
    s = O.RavenShape.nebel()
    assert (cfg.n_embd, cfg.n_heads, cfg.head_dim, cfg.intermediate_size, cfg.vocab_size) == (5280, 55, 96, 17920, 65536)
    assert cfg.effective_expected_depth == 132 and cfg.mean_recurrence == 32
    assert cfg.init_values["std"] == pytest.approx(s.init_std) and cfg.init_values["embed_scale"] == pytest.approx(s.emb_scale)
    t = pkg.RavenConfig.tiny()
    assert (t.n_embd, t.head_dim, t.n_layers_in_recurrent_block, t.mean_recurrence) == (256, 64, 2, 4)
    assert pkg.RavenConfig(**cfg.to_dict()).to_dict() == cfg.to_dict()
    with pytest.raises(ValueError):
        pkg.RavenConfig(n_embd=100, n_heads=3)


def test_remap_agrees_with_oracle(pkg):
    for strat in ("full", "latest-m4-compress-s4", "compress-s16", "compress-r4", "compress-anchor"):
        for step in list(range(0, 132)) + [-1, -2]:
            assert pkg.remap_step(step, strat) == O.remap_step(step, strat)


def test_rope_table_matches_oracle(pkg):
    assert torch.equal(pkg.precompute_freqs_cis(96, 512, 50000.0), O.rope_table(96, 512, 50000.0))


def test_cache_update_against_dict_model_on_cpu(pkg):
    """The contiguous cache driven through the reference's update() interface returns bit-identical
    K/V and the same bookkeeping as the brute-force dict model."""
    rng = torch.Generator().manual_seed(11)
    mine, ref = pkg.HuginnDynamicCache(), O.DictCache()
    for n_new in (5, 1, 1, 3):
        for step in (0, 1, 2, 3, -1, -2):
            k = torch.randn(2, 3, n_new, 8, generator=rng)
            v = torch.randn(2, 3, n_new, 8, generator=rng)
            gk, gv = mine.update(k, v, torch.tensor(step))
            wk, wv = ref.update(k, v, torch.tensor(step))
            assert torch.equal(gk, wk) and torch.equal(gv, wv)
            assert mine.get_seq_length() == ref.get_seq_length()
    assert list(mine.key_cache) == list(ref.key_cache)  # same step keys, same first-touch order
    for step in ref.key_cache:
        assert sorted(mine.key_cache[step].keys()) == sorted(ref.key_cache[step])
        for pos, t in ref.key_cache[step].items():
            assert torch.equal(mine.key_cache[step][pos], t)
            assert torch.equal(mine.value_cache[step][pos], ref.value_cache[step][pos])
    assert mine.get_memory_usage() == ref.get_memory_usage()
    mine.clear_last_k_entries(4)
    ref.clear_last_k_entries(4)
    assert mine.get_seq_length() == ref.get_seq_length() == 6
    assert all(len(mine.key_cache[s]) == len(ref.key_cache[s]) for s in ref.key_cache)
    with pytest.raises(AssertionError):
        mine.update(torch.zeros(2, 3, 1, 8), torch.zeros(2, 3, 1, 8), 2)  # overwrite of position 5 at a non-coda step
    mine.reset()
    assert mine.get_seq_length() == 0 and len(mine.key_cache) == 0


def test_cache_growth_keeps_contents_and_slot_order(pkg):
    c = pkg.HuginnDynamicCache()
    k = torch.arange(2 * 2 * 300 * 4, dtype=torch.float32).view(2, 2, 300, 4)
    c.update(k, -k, 0)
    c.update(k + 1, -k - 1, -1)
    assert c.t_max == 512
    c.update(k[:, :, :250], k[:, :, :250], 0)      # 550 tokens: storage doubles
    c.update(k[:, :, :250] + 1, k[:, :, :250], -1)
    c.update(k[:, :, :1], k[:, :, :1], 7)          # a new, higher step: slots are appended
    assert c.t_max == 1024 and c.get_seq_length() == 550
    assert torch.equal(c.key_cache[0][299], k[:, :, 299]) and torch.equal(c.key_cache[-1][0], k[:, :, 0] + 1)
    assert torch.equal(c.key_cache[0][300], k[:, :, 0]) and torch.equal(c.value_cache[-1][549], k[:, :, 249])
    fixed = pkg.HuginnDynamicCache(max_length=8)
    fixed.update(torch.zeros(1, 1, 8, 4), torch.zeros(1, 1, 8, 4), 0)
    with pytest.raises(ValueError, match="max_length"):
        fixed.update(torch.zeros(1, 1, 1, 4), torch.zeros(1, 1, 1, 4), 0)


def test_cache_capacity_keeps_head_regions_on_whole_cache_lines(pkg):
    """The storage of a head ([t_max, head_dim], contiguous) is a whole number of 128-byte lines: 192-byte rows (head_dim 96,
    bf16) get an even capacity, rows of 128 or 256 bytes any; max_length still bounds the sequence, not the storage."""
    f = pkg.cache.line_aligned_positions
    assert f(1025, 96, torch.bfloat16) == 1026 and f(1026, 96, torch.bfloat16) == 1026 and f(537, 96, torch.bfloat16) == 538
    assert f(1025, 96, torch.float32) == 1025 and f(1025, 64, torch.bfloat16) == 1025 and f(1025, 128, torch.bfloat16) == 1025
    assert f(5, 8, torch.bfloat16) == 8 and f(9, 8, torch.bfloat16) == 16          # 16-byte rows: eight to a line
    for t in range(1, 40):
        for hd, dt in ((96, torch.bfloat16), (8, torch.bfloat16), (24, torch.float32), (4, torch.float32)):
            cap = f(t, hd, dt)
            assert cap >= t and cap * hd * torch.empty((), dtype=dt).element_size() % 128 == 0 and cap - t < 128
    c = pkg.HuginnDynamicCache(max_length=7)
    c.update(torch.zeros(1, 2, 7, 96, dtype=torch.bfloat16), torch.zeros(1, 2, 7, 96, dtype=torch.bfloat16), 0)
    assert c.t_max == 8 and c.get_seq_length() == 7
    with pytest.raises(ValueError, match="max_length"):
        c.update(torch.zeros(1, 2, 1, 96, dtype=torch.bfloat16), torch.zeros(1, 2, 1, 96, dtype=torch.bfloat16), 0)


def test_cache_size_known_answers(pkg):
    """The reference notebooks' cache sizes (examples/inference_demo.ipynb:252, 373) from the
    contiguous cache's own accounting."""
    s = O.RavenShape.nebel()
    for strat, want in (("full", 973.0810546875), ("latest-m4-compress-s16", 147.4365234375)):
        c = pkg.HuginnDynamicCache(strat)
        c._k = torch.empty(1, 1, s.n_heads, 1, s.head_dim, dtype=torch.bfloat16)  # shape carrier only
        for step in O.step_indices(s):
            c.note_append(step, 366, 0)
        assert c.get_memory_usage() == want


def test_static_cache_known_answer_and_interface(pkg):
    """examples/inference_demo.ipynb:491 of the reference: 132 steps x 1 x 55 x 1024 x 96, K+V, bf16 = 2722.5 MB."""
    c = pkg.HuginnStaticCache(max_length=1024, max_num_steps=4 + 32 * 4, num_heads=55, hidden_dim=96, batch_size=1,
                              dtype=torch.bfloat16)
    assert c.get_memory_usage() == 2722.5 and c.t_max == 1024 and c.max_num_steps == 132
    k = torch.ones(1, 55, 3, 96, dtype=torch.bfloat16)
    gk, gv = c.update(k, 2 * k, torch.tensor(0))
    assert gk.shape == (1, 55, 3, 96) and c.get_seq_length() == 3
    gk, _ = c.update(k, k, torch.tensor(-1))
    assert torch.equal(gk, k) and list(c.key_cache) == [0, -1]
    s16 = pkg.HuginnStaticCache(max_length=8, max_num_steps=132, num_heads=2, hidden_dim=4, lookup_strategy="latest-m4-compress-s16")
    assert s16.max_num_steps == 20


@pytest.mark.parametrize("strategy", ["full", "skip", "latest-m4", "available-m4", "always-last-m4", "latest-m4-compress-s4",
                                      "latest-m4-compress-s16", "available-m4-compress-s8", "skip-compress-r4", "latest-m4-compress-r2",
                                      "available-m4-compress-r4", "latest-m4-compress-anchor", "skip-compress-anchor"])
def test_cache_lookups_with_partially_filled_steps_match_dict_model(pkg, strategy):
    """Tokens computed with different numbers of recurrences: every update of the contiguous cache returns what the
    brute-force dict model of the reference's cache returns (RMM:199-253), also when steps share entries (the
    compress-* remaps, RMM:169-182: a deeper token then finds shallower tokens missing at the shared entries it is
    the first to reach, and later recurrences overwrite the entries of earlier ones)."""
    g = torch.Generator().manual_seed(5)
    ours, ref = pkg.HuginnDynamicCache(strategy), O.DictCache(strategy)
    # (new tokens, recurrences): a prefill, then single tokens that stop earlier or go deeper; 9 and 11 recurrences reach
    # past the 8 recurrences compress-anchor keeps apart
    schedule = ((5, 3), (1, 1), (1, 4), (2, 2), (1, 6), (1, 3))
    if "anchor" in strategy or "compress-s16" in strategy:
        schedule += ((1, 9), (2, 5), (1, 11), (1, 8))
    for n_new, r in schedule:
        for step in [0, 1] + list(range(2, 2 + 4 * r)) + [-1, -2]:
            k, v = torch.randn(2, 3, n_new, 8, generator=g), torch.randn(2, 3, n_new, 8, generator=g)
            try:
                want = ref.update(k, v, step)
            except ValueError:
                # the reference's max() over an empty list: an older position holds no entry of this block at all (the
                # compress-r remaps put whole recurrences into single entries); the contiguous cache refuses it too
                with pytest.raises(ValueError):
                    ours.update(k, v, step)
                return
            got = ours.update(k, v, step)
            assert got[0].shape == want[0].shape, (strategy, step, got[0].shape, want[0].shape)
            assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1]), (strategy, step)
        assert ours.get_seq_length() == ref.get_seq_length()
        assert ours.get_memory_usage() == ref.get_memory_usage()
    for step in ref.key_cache:
        assert sorted(ours.key_cache[step].keys()) == sorted(ref.key_cache[step].keys()), step
    ours.clear_last_k_entries(2)
    ref.clear_last_k_entries(2)
    k = torch.randn(2, 3, 1, 8, generator=g)
    for step in [0, 1] + list(range(2, 2 + 4 * 5)):
        got, want = ours.update(k, k, step), ref.update(k, k, step)
        assert torch.equal(got[0], want[0]), (strategy, step)


@pytest.mark.parametrize("strategy", ["randomized", "randomized-compress-s4"])
def test_randomized_lookup_matches_dict_model_draw_for_draw(pkg, strategy):
    """RMM:255-271: with the CPU generator seeded alike, the contiguous cache returns the entries the dict model of the
    reference draws, and leaves the generator in the same state (one draw per position and lookup, in position order)."""
    g = torch.Generator().manual_seed(11)
    ours, ref = pkg.HuginnDynamicCache(strategy), O.DictCache(strategy)
    for i, (n_new, r) in enumerate(((4, 3), (1, 1), (1, 4), (2, 2), (1, 6), (1, 3))):
        for step in [0, 1] + list(range(2, 2 + 4 * r)) + [-1, -2]:
            k, v = torch.randn(2, 3, n_new, 8, generator=g), torch.randn(2, 3, n_new, 8, generator=g)
            torch.manual_seed(100 * i + step + 7)
            want = ref.update(k, v, step)
            state = torch.get_rng_state()
            torch.manual_seed(100 * i + step + 7)
            got = ours.update(k, v, step)
            assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1]), (strategy, i, step)
            assert torch.equal(torch.get_rng_state(), state), (strategy, i, step)


def test_cache_lookup_errors(pkg):
    c = pkg.HuginnDynamicCache("latest-m4")
    k = torch.zeros(1, 1, 1, 4)
    for step in (0, 1, 2, 3, 4, 5):
        c.update(k, k, step)
    for step in (0, 1, 2, 3, 4, 5, 6):
        c.update(k, k, step)
    c2 = pkg.HuginnDynamicCache("randomized")  # update() serves it; the kernels' descriptor does not
    for step in (0, 1, 2, 3, 4, 5):
        c2.update(k, k, step)
    for step in (0, 1, 2, 3, 4, 5, 6):
        c2.update(k, k, step)
    with pytest.raises(NotImplementedError, match="randomized"):
        pkg.cache.lookup_mode(c2.lookup_strategy)
    c3 = pkg.HuginnDynamicCache("no-such-strategy")
    for step in (0, 1, 2, 3, 4, 5, 0, 1, 2, 3, 4, 5):
        c3.update(k, k, step)
    with pytest.raises(ValueError, match="Unknown lookup strategy"):
        c3.update(k, k, 6)


# ----------------------------------------------------------------------------- committed fixtures (tests/golden)
def _golden(name):
    import json
    import os
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", name)) as f:
        return json.load(f)


def test_oracle_reproduces_the_committed_fixture():
    """tests/golden/tiny_fp32_oracle.json was written by tests/golden/make_fixtures.py: a change of the oracle's
    arithmetic, of its seeded draws or of its generate loops shows up here."""
    fx = _golden("tiny_fp32_oracle.json")
    s = O.RavenShape.tiny()
    w = O.make_weights(s, seed=0, dtype=torch.float32)
    ids = torch.tensor(fx["prompt"])
    states = O.initialize_state(torch.empty(2, 6, s.n_embd), s, 1.0, torch.Generator().manual_seed(12))
    out = O.forward(w, s, input_ids=ids, input_states=states)
    assert torch.allclose(out.logits[:, -1, :8], torch.tensor(fx["forward_last_logits_first8"]), atol=2e-5)
    assert out.logits[:, -1].argmax(-1).tolist() == fx["forward_last_argmax"]
    sf = lambda call, shape: O.initialize_state(torch.empty(shape), s, 1.0, torch.Generator().manual_seed(7000 + call))
    assert O.greedy_generate(w, s, ids, 16, state_fn=sf)[:, 6:].tolist() == fx["greedy_16_tokens"]
    toks, steps = O.generate_with_adaptive_compute(w, s, ids, 6, criterion="kl", exit_threshold=5e-3, num_steps=8, state_fn=sf,
                                                   cache_lookup_strategy="latest-m4")
    assert toks[:, 6:].tolist() == fx["adaptive_kl_5e-3_tokens"] and steps == fx["adaptive_kl_5e-3_compute_steps"]
    spec = O.generate_speculative(w, s, ids[:1], 10, draft_steps=1, lookahead_for_draft=3, num_steps=4, init_scale=0.0)
    assert spec[:, 6:].tolist() == fx["speculative_draft1_look3_tokens"]


def test_reference_published_cache_sizes_from_the_fixture(pkg):
    """The three cache sizes the reference's notebook prints, from the fixture file, against the oracle's dict cache
    and this package's two cache classes."""
    ka = _golden("reference_known_answers.json")
    s = O.RavenShape.nebel()
    for case in ka["cases"][:2]:
        c = pkg.HuginnDynamicCache(case["strategy"])
        c._k = torch.empty(1, 1, s.n_heads, 1, s.head_dim, dtype=torch.bfloat16)  # shape carrier only
        for step in O.step_indices(s):
            c.note_append(step, case["tokens"], 0)
        assert c.get_memory_usage() == case["MB"]
        d = O.DictCache(case["strategy"])
        one = torch.zeros(1, s.n_heads, 1, s.head_dim, dtype=torch.bfloat16)
        for step in O.step_indices(s):
            d.update(one.expand(1, s.n_heads, case["tokens"], s.head_dim), one.expand(1, s.n_heads, case["tokens"], s.head_dim), step)
        assert d.get_memory_usage() == case["MB"]
    static = pkg.HuginnStaticCache(max_length=1024, max_num_steps=4 + 4 * 32, num_heads=s.n_heads, hidden_dim=s.head_dim,
                                   batch_size=1, device="meta", dtype=torch.bfloat16)
    assert static.get_memory_usage() == ka["cases"][2]["MB"]


# ----------------------------------------------------------------------------- vLLM plugin naming
def test_vllm_flat_layer_names_and_schedule(pkg):
    """Hugging Face names -> the vLLM plugin's flat names (vllm/raven_vllm.py:481-526), spot values by hand, a full
    round trip over the 3.5b state-dict layout, and the order of a forward over the flat layers (raven_vllm.py:389-411)."""
    vb = pkg.vllm_binding
    cfg = pkg.RavenConfig()
    hand = {
        "transformer.wte.weight": "model.embed_tokens.weight",
        "lm_head.weight": "model.embed_tokens.weight",
        "transformer.prelude.1.attn.Wqkv.weight": "model.layers.1.self_attn.qkv_proj.weight",
        "transformer.core_block.0.mlp.fc.weight": "model.layers.2.mlp.gate_up_proj.weight",
        "transformer.core_block.3.attn.qk_bias": "model.layers.5.self_attn.qk_bias",
        "transformer.coda.1.mlp.proj.weight": "model.layers.7.mlp.down_proj.weight",
        "transformer.coda.0.attn.proj.weight": "model.layers.6.self_attn.o_proj.weight",
        "transformer.core_block.2.norm_3.weight": "model.layers.4.norm_3.weight",
        "transformer.ln_f.weight": "model.ln_f.weight",
        "transformer.adapter.weight": "model.adapter.weight",
        "freqs_cis": None,
    }
    for hf, want in hand.items():
        assert vb.vllm_name(hf, cfg) == want, hf
    names = [n for n, _ in O.state_dict_layout(O.RavenShape.nebel())]
    mapped = [vb.vllm_name(n, cfg) for n in names]
    assert len(set(mapped)) == len(names) and all(vb.hf_name(m, cfg) == n for m, n in zip(mapped, names))
    assert sum(m.startswith("model.layers.") for m in mapped) == 8 * 9
    sd = {"transformer.core_block.1.attn.qk_bias": torch.zeros(2, 1, 55, 96), "freqs_cis": torch.zeros(1), "lm_head.weight": torch.ones(3),
          "transformer.wte.weight": torch.ones(3)}
    out = vb.to_vllm_state_dict(sd, cfg)
    assert set(out) == {"model.layers.3.self_attn.qk_bias", "model.embed_tokens.weight"}
    assert out["model.layers.3.self_attn.qk_bias"].shape == (2, 55, 96)
    plan = vb.flat_layer_schedule(cfg, num_steps=2)
    assert plan == ([("layer", 0), ("layer", 1)] + [("adapter", 0)] + [("layer", i) for i in (2, 3, 4, 5)] + [("adapter", 1)]
                    + [("layer", i) for i in (2, 3, 4, 5)] + [("ln_f", 0), ("layer", 6), ("layer", 7), ("ln_f", 1)])
    assert len(vb.flat_layer_schedule(cfg)) == 2 + 32 * 5 + 1 + 2 + 1


def test_checkpoint_directory_round_trip(pkg, tmp_path):
    """from_pretrained / save_pretrained on a local directory in the layout of the reference's published checkpoints:
    config.json + safetensors (one file, or shards with an index) or pytorch_model.bin; tied head stored once; the
    parameter containers need no GPU."""
    import json
    import torch
    cfg = pkg.RavenConfig.tiny()
    model = pkg.RavenForCausalLM(cfg, device="cpu", dtype=torch.float32)
    model.init_weights(seed=3)
    want = {k: v.clone() for k, v in model.state_dict().items()}
    one, many = tmp_path / "one", tmp_path / "many"
    model.save_pretrained(str(one))
    model.save_pretrained(str(many), max_shard_bytes=600_000)
    assert (one / "model.safetensors").exists() and not (one / "model.safetensors.index.json").exists()
    index = json.loads((many / "model.safetensors.index.json").read_text())
    assert len(set(index["weight_map"].values())) > 2 and "lm_head.weight" not in index["weight_map"]
    for d in (one, many):
        got = pkg.RavenForCausalLM.from_pretrained(str(d), device="cpu", dtype=torch.float32)
        skip = ("architectures", "dtype", "torch_dtype")  # the file names the class and the dtype the weights were saved in
        assert {k: v for k, v in got.config.to_dict().items() if k not in skip} == {k: v for k, v in cfg.to_dict().items() if k not in skip}
        assert got.config.to_dict()["dtype"] == "float32" and got.config.architectures == ["RavenForCausalLM"]
        sd = got.state_dict()
        assert sd.keys() == want.keys() and all(torch.equal(sd[k], want[k]) for k in want)
        assert got.lm_head.weight.data_ptr() == got.transformer.wte.weight.data_ptr()          # still tied
    # a config override and a dtype change on load
    half = pkg.RavenForCausalLM.from_pretrained(str(one), device="cpu", dtype=torch.bfloat16, mean_recurrence=7)
    assert half.config.mean_recurrence == 7 and half.transformer.adapter.weight.dtype == torch.bfloat16
    assert torch.equal(half.transformer.adapter.weight, want["transformer.adapter.weight"].bfloat16())
    # the legacy single-file layout, read without unpickling code
    legacy = tmp_path / "legacy"
    legacy.mkdir()
    (legacy / "config.json").write_text((one / "config.json").read_text())
    torch.save({k: v for k, v in want.items() if k != "lm_head.weight"}, str(legacy / "pytorch_model.bin"))
    got = pkg.RavenForCausalLM.from_pretrained(str(legacy), device="cpu", dtype=torch.float32)
    assert all(torch.equal(got.state_dict()[k], want[k]) for k in want)
    # mismatches are errors, not silent partial loads
    from safetensors.torch import save_file
    bad = tmp_path / "bad"
    bad.mkdir()
    (bad / "config.json").write_text((one / "config.json").read_text())
    save_file({"transformer.ln_f.weight": want["transformer.ln_f.weight"], "transformer.nonsense": torch.zeros(1)}, str(bad / "model.safetensors"))
    with pytest.raises(KeyError, match="missing"):
        pkg.RavenForCausalLM.from_pretrained(str(bad), device="cpu")
    wrong = dict(cfg.to_dict(), n_embd=128, n_heads=2)
    (bad / "config.json").write_text(json.dumps(wrong))
    save_file({k: v for k, v in want.items() if k != "lm_head.weight"}, str(bad / "model.safetensors"))
    with pytest.raises(ValueError, match="shape"):
        pkg.RavenForCausalLM.from_pretrained(str(bad), device="cpu")
    with pytest.raises(FileNotFoundError):
        (tmp_path / "empty").mkdir()
        (tmp_path / "empty" / "config.json").write_text((one / "config.json").read_text())
        pkg.RavenForCausalLM.from_pretrained(str(tmp_path / "empty"), device="cpu")


def test_repetition_penalties_against_the_reference_loops(pkg):
    """The standard repetition penalty and the n-gram penalty against a literal restatement of the reference's loops
    (RMM:2003-2060, per vocabulary entry and start position) on a small vocabulary."""
    import types
    import torch
    from recurrent_pretraining_amd.sampling import apply_repetition_penalty
    g = torch.Generator().manual_seed(5)
    V = 14
    ids = torch.tensor([[3, 4, 5, 3, 4, 5, 3, 4, 9, 3, 4], [1, 1, 1, 1, 2, 2, 7, 7, 1, 1, 1]])
    logits = torch.randn(2, V, generator=g) * 3

    def brute_dry(row_logits, context, mult, base, allowed):
        out = row_logits.clone()
        n = len(context)
        for vocab_idx in range(V):
            max_match = 0
            for start in range(max(0, n - 128), n - 1):
                match = 0
                while start + match < n and match < 32 and context[start + match] == context[n - match - 1]:
                    match += 1
                if match > 0 and start + match < n and context[start + match] == vocab_idx:
                    max_match = max(max_match, match + 1)
            if max_match >= allowed:
                out[vocab_idx] -= mult * base ** (max_match - allowed)
        return out

    dry = types.SimpleNamespace(repetition_penalty=1.0, dry_multiplier=0.8, dry_base=1.75, dry_allowed_length=2)
    got = apply_repetition_penalty(logits, ids, dry)
    for b in range(2):
        assert torch.allclose(got[b], brute_dry(logits[b], ids[b].tolist(), 0.8, 1.75, 2)), b
    assert not torch.equal(got, logits)   # the sequences do repeat
    # several positions of one sequence ([T, V] logits, batch of one): every position gets the row's penalty
    multi = torch.randn(3, V, generator=g)
    got = apply_repetition_penalty(multi, ids[:1], dry)
    for t in range(3):
        assert torch.allclose(got[t], brute_dry(multi[t], ids[0].tolist(), 0.8, 1.75, 2))
    # standard penalty: seen tokens' positive logits are divided, negative ones multiplied
    std = types.SimpleNamespace(repetition_penalty=1.3, dry_multiplier=0.0)
    got = apply_repetition_penalty(logits, ids, std)
    for b in range(2):
        seen = set(ids[b].tolist())
        for v in range(V):
            x = float(logits[b, v])
            want = (x * 1.3 if x < 0 else x / 1.3) if v in seen else x
            assert abs(float(got[b, v]) - want) < 1e-6
    # with the positions' own argmax tokens added to the context
    got = apply_repetition_penalty(logits.view(2, 1, V), ids, std, use_candidates=True)
    b0 = int(logits[0].argmax())
    x = float(logits[0, b0])
    assert abs(float(got[0, 0, b0]) - (x * 1.3 if x < 0 else x / 1.3)) < 1e-6
    cfg = pkg.RavenConfig(test_time_noise=0.1, test_time_noise_type="geom")
    assert cfg.to_dict()["test_time_noise"] == 0.1 and cfg.to_dict()["test_time_noise_type"] == "geom"
    with pytest.raises(ValueError):
        pkg.RavenConfig(test_time_noise=0.1, test_time_noise_type="pink")


# ---- the transformers surface (RMM:36-112, 1066-1127, 2312-2323) --------------------------------------------------
TINY_KEYS = ("n_embd", "n_heads", "n_layers", "n_layers_in_prelude", "n_layers_in_recurrent_block", "n_layers_in_coda",
             "intermediate_size", "vocab_size", "mean_recurrence")


def test_auto_classes_resolve_huginn_raven_and_build_from_a_config(pkg, tmp_path):
    from transformers import AutoConfig, AutoModel, AutoModelForCausalLM, GenerationMixin, PretrainedConfig, PreTrainedModel
    tiny = pkg.RavenConfig.tiny()
    cfg = AutoConfig.for_model("huginn_raven", **{k: getattr(tiny, k) for k in TINY_KEYS})
    assert type(cfg) is pkg.RavenConfig and isinstance(cfg, PretrainedConfig)
    assert (cfg.hidden_size, cfg.num_attention_heads, cfg.num_hidden_layers) == (256, 4, 4)      # raven_config_minimal.py:10
    assert cfg.tie_word_embeddings is True and cfg.dtype == torch.bfloat16
    model = AutoModelForCausalLM.from_config(cfg)
    assert type(model) is pkg.RavenForCausalLM and isinstance(model, PreTrainedModel) and isinstance(model, GenerationMixin)
    assert type(AutoModel.from_config(cfg)) is pkg.RavenForCausalLM
    assert model._tied_weights_keys == {"lm_head.weight": "transformer.wte.weight"}
    assert model.lm_head.weight.data_ptr() == model.transformer.wte.weight.data_ptr()
    assert model.dtype == torch.bfloat16 and not model.training
    # the reference's initialisation (RMM:73-110): truncated at 3 std, output projections scaled down, norms one
    iv, sd = cfg.init_values, model.state_dict()
    fc = sd["transformer.core_block.0.mlp.fc.weight"].float()
    for t, std in ((sd["transformer.wte.weight"], iv["embedding"]), (sd["transformer.adapter.weight"], iv["std"]),
                   (sd["transformer.prelude.0.attn.Wqkv.weight"], iv["std"]), (fc[: fc.shape[0] // 2], iv["std"]),
                   (fc[fc.shape[0] // 2:], iv["out_proj"]), (sd["transformer.coda.0.mlp.proj.weight"], iv["out_proj"]),
                   (sd["transformer.core_block.1.attn.proj.weight"], iv["out_proj"])):
        t = t.float()
        assert abs(t.std().item() / std - 1) < 0.08 and t.abs().max().item() <= 3.02 * std and abs(t.mean().item()) < 0.1 * std
    assert torch.all(sd["transformer.ln_f.weight"] == 1) and torch.all(sd["transformer.core_block.0.attn.qk_bias"] == 0)
    # a saved directory comes back through the Auto classes with the same tensors
    model.save_pretrained(tmp_path / "ckpt")
    assert AutoConfig.from_pretrained(str(tmp_path / "ckpt")).to_dict()["n_embd"] == 256
    back = AutoModelForCausalLM.from_pretrained(str(tmp_path / "ckpt"), device_map="cpu", torch_dtype=torch.bfloat16, trust_remote_code=True)
    assert type(back) is pkg.RavenForCausalLM
    assert all(torch.equal(v, back.state_dict()[k]) for k, v in sd.items())
    # the forward needs the GPU library and says so instead of computing anything on the CPU
    with pytest.raises((pkg.hip.RavenHipError, RuntimeError)):
        model(input_ids=torch.zeros(1, 2, dtype=torch.long))


def _with_counting_forward(pkg, model, calls):
    """Replaces the forward by a stand-in that only does the cache bookkeeping and makes token (seen + S) % 7 win."""
    def forward(input_ids=None, past_key_values=None, use_cache=False, position_ids=None, num_steps=None, **kw):
        B, S = input_ids.shape
        if use_cache and past_key_values is None:
            past_key_values = pkg.HuginnDynamicCache()
        seen = past_key_values._seen_tokens if past_key_values is not None else 0
        calls.append((S, seen, None if position_ids is None else position_ids.reshape(-1)[-S:].tolist(), num_steps))
        if past_key_values is not None:
            past_key_values._seen_tokens += S
        logits = torch.zeros(B, S, model.config.vocab_size)
        logits[:, :, (seen + S) % 7] = 1.0
        return pkg.CausalLMOutputRecurrentLatents(logits=logits, past_key_values=past_key_values)
    model.forward = forward


def test_transformers_generate_drives_the_forward_one_token_at_a_time(pkg):
    """The plain generate() call is transformers' loop (RMM:1126-1127): prompt once, then one token per forward on the
    cache the forward returned, positions following the cache, keyword arguments of the forward passed through."""
    from transformers import DynamicCache
    model = pkg.RavenForCausalLM(pkg.RavenConfig.tiny(), device="cpu")
    calls = []
    _with_counting_forward(pkg, model, calls)
    ids = torch.tensor([[5, 6, 7], [8, 9, 10]])
    out = model.generate(ids, max_new_tokens=4, do_sample=False, num_steps=3)
    assert out.tolist() == [[5, 6, 7, 3, 4, 5, 6], [8, 9, 10, 3, 4, 5, 6]]
    assert calls == [(3, 0, [0, 1, 2], 3), (1, 3, [3], 3), (1, 4, [4], 3), (1, 5, [5], 3)]
    # an empty cache of transformers' own class is swapped for this package's; one that holds tokens is refused
    calls.clear()
    out = model.generate(ids, max_new_tokens=2, do_sample=False, past_key_values=DynamicCache(config=model.config))
    assert out.shape == (2, 5) and [c[:2] for c in calls] == [(3, 0), (1, 3)]

    class Used:
        def get_seq_length(self):
            return 2
    with pytest.raises(ValueError, match="empty"):
        model.prepare_inputs_for_generation(ids, past_key_values=Used(), use_cache=True)


def test_prepare_inputs_for_generation_selects_the_new_tokens(pkg):
    model = pkg.RavenForCausalLM(pkg.RavenConfig.tiny(), device="cpu")
    ids = torch.arange(10).view(2, 5)
    cache = pkg.HuginnDynamicCache()
    # transformers 4.x: the loop hands over cache positions (RMM:1100)
    got = model.prepare_inputs_for_generation(ids, past_key_values=cache, cache_position=torch.tensor([3, 4]), use_cache=True, num_steps=2)
    assert got["input_ids"].tolist() == [[3, 4], [8, 9]] and got["past_key_values"] is cache and got["num_steps"] == 2
    assert got["cache_position"].tolist() == [3, 4] and "position_ids" not in got and "attention_mask" not in got
    # transformers 5.x: the number of new tokens, and positions the loop keeps for the whole sequence
    pos = torch.arange(5).view(1, 5)
    got = model.prepare_inputs_for_generation(ids, next_sequence_length=1, past_key_values=cache, position_ids=pos, use_cache=True,
                                              attention_mask=torch.ones(2, 5))
    assert got["input_ids"].tolist() == [[4], [9]] and got["position_ids"].tolist() == [[4]] and "attention_mask" not in got
    assert got["input_ids"].is_contiguous()
    # neither: all tokens; without use_cache no cache reaches the forward
    got = model.prepare_inputs_for_generation(ids, past_key_values=cache, use_cache=False)
    assert got["input_ids"].shape == (2, 5) and got["past_key_values"] is None
    # positions given per sequence must agree between the sequences (RMM:660-665 rotates the batch with one list)
    assert model._rope_positions(3, torch.tensor([[2, 3, 4], [2, 3, 4]]), None) == [2, 3, 4]
    with pytest.raises(ValueError, match="shared"):
        model._rope_positions(3, torch.tensor([[2, 3, 4], [0, 1, 2]]), None)


def test_generate_dispatch_follows_the_reference_keywords(pkg, monkeypatch):
    """RMM:1112-1127."""
    model = pkg.RavenForCausalLM(pkg.RavenConfig.tiny(), device="cpu")
    seen = []
    for name in ("generate_with_adaptive_compute", "generate_speculative", "generate_diffusion_style", "generate_minimal"):
        monkeypatch.setattr(model, name, lambda *a, _n=name, **k: seen.append(_n))
    from transformers import GenerationMixin
    monkeypatch.setattr(GenerationMixin, "generate", lambda self, *a, **k: seen.append("transformers"))
    ids = torch.zeros(1, 2, dtype=torch.long)
    model.generate(ids, criterion="entropy-diff")
    model.generate(ids, draft_steps=2)
    model.generate(ids, headway=1)
    model.generate(ids, continuous_compute=True)
    model.generate(ids, stop_tokens=set())
    model.generate(ids, pkg.GenerationSettings(max_new_tokens=2))
    model.generate(ids, max_new_tokens=2)
    assert seen == ["generate_with_adaptive_compute", "generate_speculative", "generate_diffusion_style", "generate_minimal",
                    "generate_minimal", "generate_minimal", "transformers"]
