#!/usr/bin/env python3
"""Benchmark of the recurrent-core decode path on one MI355X.

A step is one decoded token at the nebel-raven-3.5b shape in bf16: embedding, 2 prelude blocks,
r = 32 recurrences of (adapter + 4 SandwichBlocks), 2 coda blocks, ln_f, LM head over 65536 and the
greedy argmax, with the KV cache of a 512-token prompt already resident (random-init weights, random
token ids).  Prints ONE JSON line:
  value            decoded tokens/s (whole job, one GPU, batch `--batch`, default 1)
  roofline         the dominant kernel (mlp.fc GEMV with norm prologue and SwiGLU epilogue, 47 % of a
                   token's bytes): algorithmic bytes per launch / its mean duration (HIP events on the
                   launch stream)
  core_iteration   one recurrence iteration (the unit the 70 %-of-HBM target is stated on)
  bs8, bs32        the same decode at 8 and 32 sequences, each with the roofline of its own mlp.fc kernel
  prefill          the recurrent core over 4 x 4096 prompt rows (the MFMA-bound regime): a few iterations, with the
                   roofline of its dominant kernel, the tiled mlp.fc GEMM, and of the whole iteration
  cpu_baseline     the CPU oracle on this box's host cores, on a bounded sample, scaled to tokens/s
"""

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=48)
    ap.add_argument("--warmup", type=int, default=4)
    ap.add_argument("--batch", type=int, default=1)
    ap.add_argument("--prompt", type=int, default=512)
    ap.add_argument("--recurrence", type=int, default=32)
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-iters", type=int, default=3, help="fewest timed recurrence iterations of the CPU baseline")
    ap.add_argument("--cpu-seconds", type=float, default=12.0,
                    help="the CPU baseline keeps timing iterations until this much time has been spent on them (at most 400)")
    ap.add_argument("--also-batch", type=int, action="append", default=None, metavar="B",
                    help="further batch sizes reported as sub-records bs<B> (default 8 and 32; 0 = none)")
    ap.add_argument("--prefill-iters", type=int, default=8,
                    help="core iterations timed for the 'prefill' sub-record of the default line (0 = skip)")
    ap.add_argument("--adaptive", action="store_true",
                    help="per-token adaptive compute at bs=1 with a fixed cycle of recurrences per token (a next-row measurement)")
    ap.add_argument("--paged", action="store_true",
                    help="decode over block-paged caches, --batch sequences of different lengths around --prompt (a next-row measurement)")
    ap.add_argument("--paged-layout", default="HND", choices=["NHD", "HND"])
    ap.add_argument("--prefill", action="store_true",
                    help="measure the recurrent core over a whole prompt instead (bs=4 x 4096 tokens, r iterations): MFMA-bound regime")
    ap.add_argument("--prefill-batch", type=int, default=4)
    ap.add_argument("--prefill-len", type=int, default=4096)
    ap.add_argument("--tune", action="append", default=[], metavar="KEY=VALUE",
                    help="launch-shape override passed to raven_set_tuning before the run (experiments only)")
    ap.add_argument("--attention-only", type=int, default=0, metavar="N",
                    help="with --prefill: run only N launches of the chunk attention kernel at that shape (for rocprofv3 --pmc runs)")
    ap.add_argument("--gemm-only", type=int, default=0, metavar="N",
                    help="with --prefill: launch each of the five products of a core iteration N times at the prefill shape and time it")
    ap.add_argument("--library-gemm", action="store_true",
                    help="with --prefill --gemm-only: also time torch.matmul (the vendor library) on each product's operands, as a yardstick")
    ap.add_argument("--plain-weights", action="store_true",
                    help="with --prefill: the tiled GEMMs read the weight matrices as given instead of line-aligned copies of them")
    ap.add_argument("--kernel-only", type=int, default=0, metavar="N",
                    help="run only N launches of the dominant kernel plus one 256 MiB device copy (for rocprofv3 --pmc runs)")
    return ap.parse_args()


MFMA_PEAK_TFLOPS = 2500.0  # MI355X dense bf16, published


def core_iteration_bytes(cfg, batch, t_cached, elt=2, adapter_split=False):
    """Algorithmic HBM bytes of one recurrence iteration of a decode step: every weight of the adapter and the core blocks
    once (Wqkv 3h*h, attn.proj h*h, mlp.fc 2*inter*h, mlp.proj h*inter, four norm weights, the q/k bias; adapter 2h*h),
    the cached keys and values of `t_cached` positions read once per block, and the new position's K and V written.
    adapter_split: the schedule of a call with two or more recurrences, which streams only the state half of the adapter
    (h*h) per recurrence plus the fp32 sums of the embedding half (batch*h*4); the embedding half itself is read once per
    call and is counted by the caller (`adapter_once_bytes`)."""
    h, inter, nb = cfg.n_embd, cfg.intermediate_size, cfg.n_layers_in_recurrent_block
    per_block = (3 * h * h + h * h + 2 * inter * h + h * inter + 4 * h + (2 * h if cfg.qk_bias else 0)) * elt
    adapter = (h * h * elt + batch * h * 4) if adapter_split else 2 * h * h * elt
    weights = nb * per_block + adapter
    kv_read = batch * nb * 2 * h * t_cached * elt
    kv_write = batch * nb * 2 * h * elt
    return {"weights": weights, "adapter": adapter, "kv_read": kv_read, "kv_write": kv_write, "total": weights + kv_read + kv_write}


def adapter_once_bytes(cfg, batch, elt=2):
    """What a call with the adapter split by columns reads and writes once, whatever its number of recurrences: the
    embedding half of the matrix and the fp32 sums it leaves."""
    h = cfg.n_embd
    return h * h * elt + batch * h * 4


# HBM-side bytes per launch of the tiled mlp.fc GEMM at M = 16384 from rocprofv3 --pmc (FETCH_SIZE 4,454,542 KiB x 1.99974 +
# WRITE_SIZE 600,320 KiB x 1.0, both scaled by a 256 MiB copy): 8 x the 1.14 GB of operands + output, the panel re-reads
# of 256 x 256 tiles in 8 x 4 groups per XCD.  Profiler figures, so constants, with the file that holds the readings.
TILED_FC_TRAFFIC = int(4457730 * 1024 * 1.99974 + 600320 * 1024)
TILED_FC_TRAFFIC_SOURCE = "profiles/gemm_tiled_bs4x4096_counters.txt"


def prefill_record(pkg, model, B, S, r):
    """BASELINE.json configs[4]: the recurrent core over a full prompt.  Token ids uniform over the vocabulary from seed 1,
    random-init weights; the prelude runs once (untimed), then r core iterations over all B x S rows are timed (an
    iteration costs the same whatever r is: every iteration attends over its own S keys).
    FLOPs per iteration: GEMMs 2*M*(params of adapter + 4 blocks) + causal attention 4 * 2*B*nh*hd*S*(S+1)/2 * 2.
    The dominant kernel, the tiled GEMM of mlp.fc with its SwiGLU epilogue (41 % of an iteration's FLOPs), is then
    timed alone with HIP events on the launch stream, rotating over the four core blocks' matrices."""
    import torch
    dev = torch.device("cuda:0")
    cfg = model.config
    ids = torch.randint(0, cfg.vocab_size, (B, S), generator=torch.Generator().manual_seed(1)).cuda()
    cache = pkg.HuginnDynamicCache(max_length=S)
    cache.ensure(cfg.n_layers_in_prelude + cfg.n_layers_in_recurrent_block * r, cfg.n_layers_in_coda, B, cfg.n_heads, cfg.head_dim, S,
                 torch.bfloat16, dev)  # all step slots up front: no reallocation inside the timed region
    embeds, block_idx = model.embed_inputs(ids, past_key_values=cache, use_cache=True)
    state = model.initialize_state(embeds, 1.0)
    torch.cuda.synchronize()
    print(f"prefill bench: prelude done, KV cache {cache.get_allocated_mb() / 1024:.1f} GiB, timing {r} iterations", file=sys.stderr, flush=True)
    h, inter, nh, hd = cfg.n_embd, cfg.intermediate_size, cfg.n_heads, cfg.head_dim
    M = B * S
    gemm_flops = 2.0 * M * (2 * h * h + 4 * (3 * h * h + h * h + 2 * inter * h + inter * h))
    attn_flops = 4 * (2.0 * 2.0 * B * nh * hd * S * (S + 1) / 2)
    # warm-up: one iteration on a scratch copy of the step counter (uses slots of iteration 0, overwritten below)
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    cache.lookup_strategy = "compress-s4"   # warm-up writes the same four slots the timed run starts with
    model.iterate_forward(embeds, state, block_idx=block_idx, past_key_values=cache, num_steps=1)
    cache.lookup_strategy = "full"
    cache._filled = {k: v for k, v in cache._filled.items() if k < cfg.n_layers_in_prelude}
    cache._core = type(cache._core)()   # forget the warm-up's core steps: the timed run writes them again
    torch.cuda.synchronize()
    a.record()
    model.iterate_forward(embeds, state, block_idx=block_idx, past_key_values=cache, num_steps=r)
    b.record()
    torch.cuda.synchronize()
    ms = a.elapsed_time(b)
    del cache, embeds, state
    torch.cuda.empty_cache()
    tflops = (gemm_flops + attn_flops) * r / (ms * 1e-3) / 1e12
    # the dominant kernel alone
    lib = pkg.hip.load()
    stream = torch.cuda.current_stream().cuda_stream
    blocks = model.transformer.core_block
    x = torch.randn(M, h, device=dev, dtype=torch.bfloat16)
    gate = torch.empty(M, inter, device=dev, dtype=torch.bfloat16)

    def fc_launch(i=[0]):
        blk = blocks[i[0] % len(blocks)]
        i[0] += 1
        lib.raven_gemm_swiglu(x.data_ptr(), blk.mlp.fc.weight.data_ptr(), gate.data_ptr(), M, inter, h, pkg.hip.BF16, stream)

    fc_ms = event_time_ms(fc_launch, 8, warm=2)
    fc_flops = 2.0 * M * 2 * inter * h
    fc_tflops = fc_flops / (fc_ms * 1e-3) / 1e12
    return {
        "value": round(M * r / (ms * 1e-3), 1), "unit": "tokens*iterations/s", "steps": r, "warmup": 1, "ms_per_step": round(ms / r, 3),
        "config": {"workload": f"recurrent-core prefill, nebel-raven-3.5b shape, bs={B} x {S} tokens, {r} timed iterations "
                               f"(BASELINE.json configs[4])",
                   "batch": B, "seq_len": S, "iterations": r, "gemm": "gemm_ring_kernel (hand-written MFMA, 256 x 256 tiles, four waves, operands global -> LDS ring)",
                   "attention": "attention_prefill_kernel",
                   "weights": ("Wqkv, attn.proj, mlp.fc read through line-aligned copies made once (raven_register_packed_weight)"
                               if model.pack_chunk_weights else "as loaded")},
        "roofline": {"bound": "mfma", "kernel": f"gemm_ring_kernel<SwiGLU> 256x256 (mlp.fc {2 * inter}x{h}, M={M})",
                     "achieved": round(fc_tflops, 1), "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(fc_tflops / MFMA_PEAK_TFLOPS, 4), "flops_per_launch": fc_flops, "avg_us": round(fc_ms * 1e3, 1),
                     "traffic": TILED_FC_TRAFFIC, "traffic_source": TILED_FC_TRAFFIC_SOURCE},
        "iteration_roofline": {"bound": "mfma", "achieved": round(tflops, 1), "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                               "frac": round(tflops / MFMA_PEAK_TFLOPS, 4), "flops_per_iteration": gemm_flops + attn_flops},
    }


def prefill(args):
    """The configs[4] measurement as a line of its own: --recurrence iterations (32) instead of the default line's few."""
    import torch
    import __graft_entry__ as entry
    pkg = entry.import_package()
    pkg.hip.load()
    model = pkg.RavenForCausalLM(pkg.RavenConfig(), device=torch.device("cuda:0"), dtype=torch.bfloat16)
    fill_synthetic(model, 0)
    model.pack_chunk_weights = not args.plain_weights
    rec = prefill_record(pkg, model, args.prefill_batch, args.prefill_len, args.recurrence)
    line = {"metric": "core prefill tokens*iterations/s, raven-3.5b shape bf16; MFMA utilisation", "value": rec["value"],
            "unit": rec["unit"], "n_gpus": 1, "steps": rec["steps"], "warmup": rec["warmup"], "ms_per_step": rec["ms_per_step"],
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
            "config": rec["config"], "roofline": rec["roofline"], "iteration_roofline": rec["iteration_roofline"]}
    print(json.dumps(line))


def adaptive(args):
    """Per-token adaptive compute at bs=1 (next-row measurement, not the headline line): tokens stop after a fixed
    cycle of 8 / 16 / 32 / 12 recurrences (a NumStepsGenerator, so the work does not depend on what random weights
    predict), the cache lookup is latest-m4, i.e. deeper tokens read shallower tokens' last recurrence through the
    attention kernel's steps_present path.  Each recurrence is one eager raven_core_iteration call."""
    import torch
    import __graft_entry__ as entry
    pkg = entry.import_package()
    pkg.hip.load()
    dev = torch.device("cuda:0")
    cfg = pkg.RavenConfig()
    model = pkg.RavenForCausalLM(cfg, device=dev, dtype=torch.bfloat16)
    fill_synthetic(model, 0)
    sched = [8, 16, 32, 12]
    n_new = args.steps
    ids = torch.randint(0, cfg.vocab_size, (1, args.prompt), generator=torch.Generator().manual_seed(1)).cuda()
    gc = pkg.GenerationSettings(max_new_tokens=n_new + 1, return_dict_in_generate=True)
    ev = pkg.NumStepsGenerator(lambda i: 32 if i == 0 else sched[(i - 1) % len(sched)])
    # the prompt (token step 0, all 32 recurrences) is part of the call; time it separately and subtract
    for _ in range(2):  # the first pass warms up (allocations, lazy initialisation)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        model.generate_with_adaptive_compute(ids, pkg.GenerationSettings(max_new_tokens=1, return_dict_in_generate=True),
                                             exit_evaluator=pkg.NumStepsGenerator(lambda i: 32), num_steps=32,
                                             cache_lookup_strategy="latest-m4", stop_tokens=set())
        torch.cuda.synchronize()
        t_prompt = time.perf_counter() - t0
    t0 = time.perf_counter()
    out = model.generate_with_adaptive_compute(ids, gc, exit_evaluator=ev, num_steps=32, cache_lookup_strategy="latest-m4",
                                               stop_tokens=set())
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0 - t_prompt
    steps = [s_[0] for s_ in out.scores["compute_steps"]][1:]
    line = {
        "metric": "adaptive-compute decode, raven-3.5b shape bf16 bs=1: tokens/s and recurrences/s",
        "value": round(len(steps) / dt, 3), "unit": "tokens/s", "n_gpus": 1, "steps": len(steps), "warmup": 0,
        "ms_per_step": round(dt / len(steps) * 1e3, 3), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"generate_with_adaptive_compute, nebel-raven-3.5b shape, bs=1, {args.prompt}-token prompt, "
                               f"recurrences per token cycle {sched}, cache lookup latest-m4", "schedule": sched},
        "recurrences_per_s": round(sum(steps) / dt, 1), "mean_recurrences": round(sum(steps) / len(steps), 2),
        "ms_per_recurrence_incl_coda_and_head": round(dt / sum(steps) * 1e3, 4), "prompt_s": round(t_prompt, 3),
    }
    print(json.dumps(line))


def paged(args):
    """Decode steps over block-paged caches (one per flat layer, 16 positions per block, shuffled block tables), the
    sequences of the batch at different lengths drawn uniformly from [prompt / 2, 3 prompt / 2].  The pages hold
    synthetic keys and values (N(0, 1)); every step appends one position per sequence and feeds back the greedy token."""
    import torch
    import __graft_entry__ as entry
    pkg = entry.import_package()
    pkg.hip.load()
    dev = torch.device("cuda:0")
    cfg = pkg.RavenConfig()
    model = pkg.RavenForCausalLM(cfg, device=dev, dtype=torch.bfloat16)
    fill_synthetic(model, 0)
    B, bs, r = args.batch, 16, args.recurrence
    g = torch.Generator().manual_seed(1)
    lens = torch.randint(args.prompt // 2, args.prompt * 3 // 2 + 1, (B,), generator=g, dtype=torch.int32)
    total = args.steps + args.warmup
    max_blocks = (int(lens.max()) + total + bs - 1) // bs
    n_blocks = B * max_blocks
    table = torch.randperm(n_blocks, generator=g).view(B, max_blocks).to(torch.int32).to(dev)
    dec = pkg.PagedDecoder(model, num_blocks=n_blocks, block_size=bs, num_steps=r, use_graph=not args.no_graph, layout=args.paged_layout)
    # prompt processing on the pages first: up to four prompts of --prompt tokens in one forward_tokens call
    n_p, n_tok = min(B, 4), min(args.prompt, int(lens.min()))
    p_ids = torch.randint(0, cfg.vocab_size, (n_p * n_tok,), generator=g).to(dev)
    p_pos = torch.arange(n_tok).repeat(n_p)
    p_slots = torch.cat([table[b].cpu().to(torch.int64)[torch.arange(n_tok) // bs] * bs + torch.arange(n_tok) % bs for b in range(n_p)])
    p_args = (p_ids, p_pos.to(dev), p_slots.to(dev), table[:n_p], torch.full((n_p,), n_tok, dtype=torch.int32, device=dev),
              (torch.arange(n_p + 1, dtype=torch.int32) * n_tok).to(dev), n_tok)
    p_state = torch.zeros(n_p * n_tok, cfg.n_embd, dtype=torch.bfloat16, device=dev)
    dec.forward_tokens(*p_args, input_states=p_state)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    dec.forward_tokens(*p_args, input_states=p_state)
    torch.cuda.synchronize()
    prompt_dt = time.perf_counter() - t0
    for t in dec.k + dec.v:
        t.normal_(0.0, 1.0)
    ids = torch.randint(0, cfg.vocab_size, (B,), generator=g).to(dev)
    seq_lens = (lens + 1).to(dev)
    nxt = torch.zeros(B, dtype=torch.int64, device=dev)
    state = torch.zeros(B, cfg.n_embd, dtype=torch.bfloat16, device=dev)

    def one():
        state.normal_(0.0, 0.632)  # a fresh latent state per token, as the reference draws it (scale of its default initialisation)
        logits, _ = dec.step(ids, table, seq_lens, input_states=state, check_bounds=False)  # the bench builds table and lengths itself
        pkg.hip.argmax(logits, out=nxt)
        ids.copy_(nxt)
        seq_lens.add_(1)

    for _ in range(args.warmup):
        one()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        one()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    mean_len = float(lens.float().mean()) + args.warmup + args.steps / 2
    n_flat, core = dec.n_flat, cfg.n_layers_in_recurrent_block
    kv_bytes = B * mean_len * cfg.n_embd * 2 * 2 * (n_flat - core + core * r)  # K and V of every attention call of a step
    line = {
        "metric": "paged-KV decode, raven-3.5b shape bf16: tokens/s over sequences of different lengths",
        "value": round(B * args.steps / dt, 2), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(dt / args.steps * 1e3, 3), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"PagedDecoder.step, nebel-raven-3.5b shape, r={r}, {B} sequences, lengths {int(lens.min())}..{int(lens.max())} "
                               f"(mean {float(lens.float().mean()):.0f}), block size {bs}", "batch": B, "recurrence": r, "hip_graph": not args.no_graph,
                   "layout": args.paged_layout},
        "kv_GB_per_step": round(kv_bytes / 1e9, 2),
        "prompt_chunks": {"call": "PagedDecoder.forward_tokens", "sequences": n_p, "rows": n_p * n_tok, "ms": round(prompt_dt * 1e3, 2),
                          "prompt_tokens_per_s": round(n_p * n_tok / prompt_dt, 1)},
    }
    print(json.dumps(line))


def attention_only(args):
    """The chunk attention kernel alone at the prefill shape (--prefill-batch sequences of --prefill-len rows, 55 heads of
    96): synthetic q, K, V ~ N(0, 1) in a contiguous cache of one step slot; HIP events around --attention-only launches."""
    import torch
    import __graft_entry__ as entry
    pkg = entry.import_package()
    pkg.hip.load()
    cfg = pkg.RavenConfig()
    dev = torch.device("cuda:0")
    B, S, nh, hd = args.prefill_batch, args.prefill_len, cfg.n_heads, cfg.head_dim
    torch.manual_seed(0)
    k = torch.randn(1, B, nh, S, hd, device=dev, dtype=torch.bfloat16)
    v = torch.randn_like(k)
    kv = pkg.hip.make_cache(k, v)
    q = torch.randn(B * S, nh * hd, device=dev, dtype=torch.bfloat16)
    ms = event_time_ms(lambda: pkg.hip.prefill_attention(q, kv, 0, B, S, 0, nh, hd), args.attention_only, warm=2)
    flops = 4.0 * B * nh * hd * S * (S + 1) / 2
    print(json.dumps({"attention_only": args.attention_only, "kernel": "attention_prefill_kernel", "batch": B, "seq_len": S,
                      "ms_per_launch": round(ms, 4), "causal_flops_per_launch": flops, "TFLOP/s": round(flops / ms / 1e9, 1),
                      "frac_of_mfma_peak": round(flops / ms / 1e9 / MFMA_PEAK_TFLOPS, 4)}))


def gemm_only(args):
    """The five products of one core iteration alone at the prefill shape (--prefill-batch x --prefill-len token rows):
    synthetic operands, HIP events around --gemm-only launches of each, the four core blocks' worth of weights rotated so
    that no launch finds its matrix in a cache."""
    import torch
    import __graft_entry__ as entry
    pkg = entry.import_package()
    pkg.hip.load()
    cfg = pkg.RavenConfig()
    dev = torch.device("cuda:0")
    M, h, inter = args.prefill_batch * args.prefill_len, cfg.n_embd, cfg.intermediate_size
    torch.manual_seed(0)

    def mats(n, k):
        return [torch.randn(n, k, device=dev, dtype=torch.bfloat16) * 0.02 for _ in range(4)]

    x, e, res = (torch.randn(M, h, device=dev, dtype=torch.bfloat16) for _ in range(3))
    g = torch.randn(M, inter, device=dev, dtype=torch.bfloat16)
    cases = [("mlp.fc + SwiGLU", mats(2 * inter, h), dict(x=x, swiglu=True)), ("attn.Wqkv", mats(3 * h, h), dict(x=x)),
             ("attn.proj + residual", mats(h, h), dict(x=x, residual=res)), ("mlp.proj + residual", mats(h, inter), dict(x=g, residual=res)),
             ("adapter (two K segments)", mats(h, 2 * h), dict(x=x, x1=e))]
    out = {"gemm_only": args.gemm_only, "kernel": "gemm_ring_kernel / gemm_tiled_kernel", "rows": M, "products": {},
           "weights": "as given ([N, K] rows K elements apart)" if args.plain_weights else
                      "line-aligned copies (raven_register_packed_weight) of the matrices with K = 5280, as the model makes them for prompt chunks"}
    total_ms, total_flops = 0.0, 0.0
    keep = []
    for name, ws, kw in cases:
        xin = kw.pop("x")
        if not args.plain_weights and (ws[0].shape[1] * 2) % 128 != 0:
            keep += [pkg.hip.register_packed_weight(w) for w in ws]

        def launch(i=[0]):
            i[0] += 1
            pkg.hip.linear(xin, ws[i[0] % 4], **kw)

        ms = event_time_ms(launch, args.gemm_only, warm=2)
        flops = 2.0 * M * ws[0].shape[0] * ws[0].shape[1]
        n_iter = 1 if name.startswith("adapter") else 4
        total_ms += n_iter * ms
        total_flops += n_iter * flops
        out["products"][name] = {"N": ws[0].shape[0], "K": ws[0].shape[1], "ms": round(ms, 4), "TFLOP/s": round(flops / ms / 1e9, 1),
                                 "frac_of_mfma_peak": round(flops / ms / 1e9 / MFMA_PEAK_TFLOPS, 4)}
        if args.library_gemm and "x1" not in kw:
            # the same product without its epilogue through torch.matmul (the vendor library), same process and operands:
            # a yardstick beside the figure above, never part of it
            def lib_launch(i=[0]):
                i[0] += 1
                torch.matmul(xin, ws[i[0] % 4].t())

            lib_ms = event_time_ms(lib_launch, args.gemm_only, warm=2)
            out["products"][name]["library_matmul_no_epilogue"] = {"ms": round(lib_ms, 4), "TFLOP/s": round(flops / lib_ms / 1e9, 1)}
            if (ws[0].shape[1] * 2) % 128 != 0:  # and with the weight rows a whole number of lines apart, as the packed copies are
                K, ld = ws[0].shape[1], (ws[0].shape[1] + 63) // 64 * 64
                padded = []
                for w in ws:
                    wp = torch.zeros(w.shape[0], ld, device=dev, dtype=w.dtype)
                    wp[:, :K] = w
                    padded.append(wp[:, :K])

                def lib_padded(i=[0]):
                    i[0] += 1
                    torch.matmul(xin, padded[i[0] % 4].t())

                lib_ms = event_time_ms(lib_padded, args.gemm_only, warm=2)
                out["products"][name]["library_matmul_padded_rows"] = {"ms": round(lib_ms, 4), "TFLOP/s": round(flops / lib_ms / 1e9, 1)}
                del padded
    out["per_iteration"] = {"ms": round(total_ms, 3), "TFLOP/s": round(total_flops / total_ms / 1e9, 1)}
    for _, ws, _ in cases:
        for w in ws:
            pkg.hip.unregister_packed_weight(w)
    print(json.dumps(out))


def kernel_only(n_launches, batch=1):
    """The dominant kernel alone, as the decode loop launches it at `batch` sequences, on four rotating fc matrices,
    followed by one device copy of known size (the yardstick that scales FETCH_SIZE / WRITE_SIZE readings)."""
    import torch
    import __graft_entry__ as entry
    pkg = entry.import_package()
    lib = pkg.hip.load()
    cfg = pkg.RavenConfig()
    dev = torch.device("cuda:0")
    h, inter = cfg.n_embd, cfg.intermediate_size
    torch.manual_seed(0)
    fcs = [torch.randn(2 * inter, h, device=dev, dtype=torch.bfloat16) * 0.02 for _ in range(4)]
    na, nb = (torch.ones(h, device=dev, dtype=torch.bfloat16) for _ in range(2))
    x = torch.randn(batch, h, device=dev, dtype=torch.bfloat16)
    x2, g = torch.empty_like(x), torch.empty(batch, inter, device=dev, dtype=torch.bfloat16)
    stream = torch.cuda.current_stream().cuda_stream
    hp, wptrs = h, [w.data_ptr() for w in fcs]
    if 17 <= batch <= 32 and h % 64 != 0:   # as the decode step runs it at these row counts: operands with rows of whole cache lines
        hp = (h + 63) // 64 * 64
        copies = [pkg.hip.register_packed_weight(w) for w in fcs]
        wptrs = [c.data_ptr() for c in copies]
        xp = torch.zeros(batch, hp, device=dev, dtype=torch.bfloat16)
        xp[:, :h] = x
        x = xp
    for i in range(n_launches):
        if batch == 1:
            lib.raven_gemv_fused(x.data_ptr(), None, na.data_ptr(), nb.data_ptr(), x2.data_ptr(), fcs[i % 4].data_ptr(), None,
                                 g.data_ptr(), inter, h, 0, cfg.norm_eps, 1, 0, pkg.hip.BF16, stream)
        else:
            lib.raven_gemm_swiglu(x.data_ptr(), wptrs[i % 4], g.data_ptr(), batch, inter, hp, pkg.hip.BF16, stream)
    torch.cuda.synchronize()
    if hp != h:
        for w in fcs:
            pkg.hip.unregister_packed_weight(w)
    src = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
    dst = torch.empty_like(src)
    dst.copy_(src)
    torch.cuda.synchronize()
    print(json.dumps({"kernel_only": n_launches, "batch": batch, "bytes_per_launch": 2 * inter * h * 2 + batch * h * 2 + batch * inter * 2,
                      "copy_bytes": src.numel()}))


def event_time_ms(fn, reps, warm=3):
    import torch
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(reps):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / reps


def fill_synthetic(model, seed=0):
    """Random-init weights N(0, 0.02) (norm weights N(1, 0.02)) drawn on the GPU: synthetic data."""
    import torch
    torch.manual_seed(seed)
    with torch.no_grad():
        for name, p in model.state_dict().items():
            if name == "freqs_cis" or (name == "lm_head.weight" and model.config.tie_embeddings):
                continue
            p.normal_(1.0 if p.dim() == 1 else 0.0, 0.02)


def decode_tokens_per_s(pkg, model, batch, prompt_len, steps, warmup, r, use_graph):
    """Prefills a random prompt, then times `steps` greedy decode steps (state re-drawn per token)."""
    import torch
    cfg = model.config
    g = torch.Generator().manual_seed(1)
    prompt = torch.randint(0, cfg.vocab_size, (batch, prompt_len), generator=g).cuda()
    total = prompt_len + warmup + steps + 1
    cache = pkg.HuginnDynamicCache(max_length=total)
    t0 = time.perf_counter()
    out = model(input_ids=prompt, past_key_values=cache, use_cache=True, cache_position=torch.arange(prompt_len).cuda(), num_steps=r)
    torch.cuda.synchronize()
    prefill_s = time.perf_counter() - t0
    tok = out.logits[:, -1].argmax(-1)
    runner = pkg.DecodeRunner(model, cache, batch, r, greedy=True, use_graph=use_graph)
    for _ in range(warmup):
        _, nxt, _ = runner.step(tok, None, 1.0)
        tok = nxt.clone()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        _, nxt, _ = runner.step(tok, None, 1.0)
        tok = nxt.clone()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    return batch * steps / dt, dt / steps * 1e3, prefill_s, cache


def apply_tuning(args):
    if not args.tune:
        return
    import __graft_entry__ as entry
    hip = entry.import_package().hip
    for item in args.tune:
        key, value = item.split("=")
        hip.set_tuning(key, int(value))


def main():
    args = parse()
    apply_tuning(args)
    if args.kernel_only:
        kernel_only(args.kernel_only, args.batch)
        return
    if args.prefill and args.attention_only:
        attention_only(args)
        return
    if args.prefill and args.gemm_only:
        gemm_only(args)
        return
    if args.prefill:
        prefill(args)
        return
    if args.adaptive:
        adaptive(args)
        return
    if args.paged:
        paged(args)
        return
    if args.gpus != 1:
        print("bench.py measures one GPU: the decode path has no multi-GPU part (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    import torch
    import __graft_entry__ as entry

    pkg = entry.import_package()
    pkg.hip.load()
    assert torch.cuda.is_available(), "bench.py needs the GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    cfg = pkg.RavenConfig()
    r = args.recurrence
    model = pkg.RavenForCausalLM(cfg, device=dev, dtype=torch.bfloat16)
    fill_synthetic(model, 0)
    use_graph = not args.no_graph
    h = cfg.n_embd
    lib = pkg.hip.load()
    stream = torch.cuda.current_stream().cuda_stream

    head = decode_record(pkg, model, args.batch, args.prompt, args.steps, args.warmup, r, use_graph)
    tok_s, ms_step = head["tokens_per_s"], head["ms_per_step"]

    # ---- device copy bandwidth, for context next to the published peak ----
    src = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
    dst = torch.empty_like(src)
    copy_ms = event_time_ms(lambda: dst.copy_(src), 10)
    copy_gbs = 2 * src.numel() / (copy_ms * 1e-3) / 1e9
    del src, dst

    # ---- the isolated norm kernel (BASELINE.json configs[1]): x + residual -> RMSNorm, [T, 5280] bf16, 31,680 B per row ----
    norm_w = model.transformer.core_block[0].norm_1.weight
    norm_cfg2 = {}
    for T_rows in (1, 32, 4096):
        xs = [torch.randn(T_rows, h, device=dev, dtype=torch.bfloat16) for _ in range(8)]  # rotate: 8 x 43 MB at T = 4096
        rs = torch.randn(T_rows, h, device=dev, dtype=torch.bfloat16)
        yo = torch.empty_like(rs)

        def norm_launch(i=[0]):
            i[0] += 1
            lib.raven_rmsnorm_residual(xs[i[0] % 8].data_ptr(), rs.data_ptr(), norm_w.data_ptr(), yo.data_ptr(), None, None, None, T_rows, h,
                                       cfg.norm_eps, pkg.hip.BF16, stream)

        t_ms = event_time_ms(norm_launch, 100, warm=10)
        norm_cfg2[f"T={T_rows}"] = {"us": round(t_ms * 1e3, 2), "GBs": round(T_rows * 3 * h * 2 / (t_ms * 1e-3) / 1e9, 1)}
        del xs, rs, yo

    subs = {}
    for b2 in ([8, 32] if args.also_batch is None else args.also_batch):
        if b2 and b2 != args.batch:
            torch.cuda.empty_cache()
            subs[f"bs{b2}"] = decode_record(pkg, model, b2, args.prompt, max(8, args.steps // 4), 2, r, use_graph)

    pre = None
    if args.prefill_iters:
        torch.cuda.empty_cache()
        pre = prefill_record(pkg, model, args.prefill_batch, args.prefill_len, args.prefill_iters)

    cpu = None
    if not args.no_cpu_baseline:
        cpu = cpu_baseline(model, args.cpu_iters, r, args.cpu_seconds)

    line = {
        "metric": "decode tokens/s at r=32, raven-3.5b shape bf16 bs=1/32; % HBM roofline",
        "value": round(tok_s, 3),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": f"full-token greedy decode, nebel-raven-3.5b shape, r={r}, bs={args.batch}, "
                               f"{args.prompt}-token random prompt, {args.steps} timed tokens (BASELINE.json configs[3])",
                   "batch": args.batch, "recurrence": r, "prompt": args.prompt, "hip_graph": use_graph},
        "recurrence_steps_per_s": head["recurrence_steps_per_s"],
        "token_roofline": head["token_roofline"],
        "roofline": head["roofline"],
        "core_iteration": head["core_iteration"],
        "rmsnorm_residual_5280": norm_cfg2,
        "device_copy_GBs": round(copy_gbs, 1),
        "prefill_s": head["prefill_s"],
        **subs,
        "prefill": pre,
        "cpu_baseline": cpu,
    }
    print(json.dumps(line))


# HBM bytes per launch of the mlp.fc kernel from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by a 256 MiB copy: profiler
# figures, so constants here, with the file that holds the readings
FC_TRAFFIC = {1: 385924535, 8: 382192138, 32: 386341464}
FC_TRAFFIC_SOURCE = "profiles/mlp_fc_decode_hbm_traffic.txt"


def decode_record(pkg, model, B, prompt_len, steps, warmup, r, use_graph):
    """Full-token decode at B sequences with what bounds it: tokens/s over `steps` greedy tokens, one recurrence
    iteration at 1024 cached positions (single eager calls, and a replayed graph of a token's worth of them, each leg over
    the bytes its own schedule streams and over distinct K/V slots), and the dominant kernel -- the
    mlp.fc product with its norm prologue and SwiGLU epilogue, 47 % of a token's bytes -- alone, timed with HIP events on
    the launch stream exactly as the decode loop launches it, rotating over the four core blocks' fc matrices (1.5 GB)
    so that no cache level can keep a matrix between launches."""
    import torch
    cfg = model.config
    dev = model.device
    tok_s, ms_step, prefill_s, cache = decode_tokens_per_s(pkg, model, B, prompt_len, steps, warmup, r, use_graph)
    del cache
    torch.cuda.empty_cache()
    mean_t = prompt_len + warmup + steps / 2.0
    # a token's r recurrences are one library call, which splits the adapter by columns (state half per recurrence, embedding
    # half once per token) whenever r >= 2: count what that schedule streams
    split = r >= 2
    bb = core_iteration_bytes(cfg, B, int(mean_t), adapter_split=split)
    per_block_w = (bb["weights"] - bb["adapter"]) // 4
    token_bytes = (r * bb["total"] + (adapter_once_bytes(cfg, B) if split else 0)
                   + 4 * (per_block_w + (bb["kv_read"] + bb["kv_write"]) // 4) + cfg.vocab_size * cfg.n_embd * 2)

    # ---- one recurrence iteration at T = 1024 (the unit of the roofline target) ----
    # Two legs, each with the bytes its own schedule streams: (1) single raven_core_iteration launches (whole adapter per
    # iteration); (2) a replayed HIP graph of one raven_core_iterations call of n_it recurrences, as the decode loop
    # issues them (adapter split by columns, its embedding half read once per call).  Both walk distinct K/V slots, as a
    # token's recurrences do: 128 slots (2.8 GB) for one sequence, 32 slots for more.
    h, nh, hd, T = cfg.n_embd, cfg.n_heads, cfg.head_dim, 1024
    nat = model._natives()
    n_slots = 128 if B == 1 else 32
    n_it = n_slots // 4
    t_cap = pkg.cache.line_aligned_positions(T + 1, hd, torch.bfloat16)   # the capacity HuginnDynamicCache allocates for T + 1 positions
    kc = torch.empty(n_slots, B, nh, t_cap, hd, device=dev, dtype=torch.bfloat16).normal_()
    vc = torch.empty(n_slots, B, nh, t_cap, hd, device=dev, dtype=torch.bfloat16).normal_()
    kv = pkg.hip.make_cache(kc, vc)
    ws = pkg.hip.block_workspace(nat["dims"], B, dev)
    state = torch.randn(B, h, device=dev, dtype=torch.bfloat16)
    emb = torch.randn(B, h, device=dev, dtype=torch.bfloat16)
    outb = torch.empty_like(state)
    adapter_w = model.transformer.adapter.weight

    def one_iter(i=[0]):
        i[0] += 1
        pkg.hip.core_iteration(nat["dims"], adapter_w, nat["core"], state, emb, outb, nat["freqs"], kv, 4 * (i[0] % n_it), B, 1, T, ws)

    def many_iters():
        pkg.hip.core_iterations(nat["dims"], adapter_w, nat["core"], state, emb, outb, nat["freqs"], kv,
                                [[4 * it + j for j in range(4)] for it in range(n_it)], B, 1, T, ws)

    iter_eager_ms = event_time_ms(one_iter, 2 * n_it, warm=n_it)
    many_iters()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        many_iters()
    iter_graph_ms = event_time_ms(graph.replay, 6, warm=2) / n_it
    eager_bytes = core_iteration_bytes(cfg, B, T)["total"]
    graph_bytes = core_iteration_bytes(cfg, B, T, adapter_split=True)["total"] + adapter_once_bytes(cfg, B) / n_it
    eager_gbs = eager_bytes / (iter_eager_ms * 1e-3) / 1e9
    graph_gbs = graph_bytes / (iter_graph_ms * 1e-3) / 1e9
    del graph, kc, vc, kv

    # ---- dominant kernel ----
    blocks = model.transformer.core_block
    xin = torch.randn(B, h, device=dev, dtype=torch.bfloat16)
    x2 = torch.empty_like(xin)
    gout = torch.empty(B, cfg.intermediate_size, device=dev, dtype=torch.bfloat16)
    lib = pkg.hip.load()
    stream = torch.cuda.current_stream().cuda_stream
    if B == 1:
        kernel_name = "gemv1_kernel<bf16, C=3, SwiGLU, norm prologue, 7 row pairs per workgroup> (mlp.fc 35840x5280)"

        def fc_launch(i=[0]):
            blk = blocks[i[0] % len(blocks)]
            i[0] += 1
            lib.raven_gemv_fused(xin.data_ptr(), None, blk.norm_2.weight.data_ptr(), blk.norm_3.weight.data_ptr(), x2.data_ptr(),
                                 blk.mlp.fc.weight.data_ptr(), None, gout.data_ptr(), cfg.intermediate_size, h, 0, cfg.norm_eps, 1, 0,
                                 pkg.hip.BF16, stream)
    else:
        kernel_name = "mfma_kernel<SwiGLU> (mlp.fc 35840x5280)" if B > 4 else "gemv_kernel<bf16, SwiGLU> (mlp.fc 35840x5280)"

        # 17..32 rows: the decode step runs this product over line-aligned operands (the model's registered copies of the
        # matrices, x with zero-padded rows), so that is what is timed; the bytes stay the algorithmic ones
        copies = {w.data_ptr(): buf for w, buf in model._packed.ptr_owner}
        padded = 17 <= B <= 32 and h % 64 != 0 and all(blk.mlp.fc.weight.data_ptr() in copies for blk in blocks)
        hp = (h + 63) // 64 * 64 if padded else h
        if padded:
            kernel_name += ", rows padded to whole cache lines"
            xp = torch.zeros(B, hp, device=dev, dtype=torch.bfloat16)
            xp[:, :h] = xin
            xin = xp

        def fc_launch(i=[0]):
            blk = blocks[i[0] % len(blocks)]
            i[0] += 1
            wptr = copies[blk.mlp.fc.weight.data_ptr()].data_ptr() if padded else blk.mlp.fc.weight.data_ptr()
            lib.raven_gemm_swiglu(xin.data_ptr(), wptr, gout.data_ptr(), B, cfg.intermediate_size, hp, pkg.hip.BF16, stream)

    fc_ms = event_time_ms(fc_launch, 200, warm=10)
    fc_bytes = blocks[0].mlp.fc.weight.numel() * 2 + B * h * 2 + B * cfg.intermediate_size * 2
    fc_gbs = fc_bytes / (fc_ms * 1e-3) / 1e9
    return {
        "batch": B, "tokens_per_s": round(tok_s, 3), "ms_per_step": round(ms_step, 4), "steps": steps, "prefill_s": round(prefill_s, 3),
        "recurrence_steps_per_s": round(tok_s * r / B, 2),
        "token_roofline": {"bytes_per_token": int(token_bytes), "adapter_split": split, "achieved_GBs": round(token_bytes * (tok_s / B) / 1e9, 1),
                           "frac": round(token_bytes * (tok_s / B) / 1e9 / HBM_PEAK_GBS, 4)},
        "roofline": {"bound": "hbm", "kernel": kernel_name,
                     "achieved": round(fc_gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(fc_gbs / HBM_PEAK_GBS, 4),
                     "bytes_per_launch": int(fc_bytes), "avg_us": round(fc_ms * 1e3, 2),
                     "traffic": FC_TRAFFIC.get(B), "traffic_source": FC_TRAFFIC_SOURCE if B in FC_TRAFFIC else None},
        # frac is the graph leg's: the schedule the decode loop runs, over the bytes that schedule streams
        "core_iteration": {"T": T, "batch": B, "kv_slots_walked": n_slots,
                           "eager_single_call": {"bytes": int(eager_bytes), "ms": round(iter_eager_ms, 4), "achieved_GBs": round(eager_gbs, 1),
                                                 "frac": round(eager_gbs / HBM_PEAK_GBS, 4), "adapter": "whole (2h x h) per iteration"},
                           "graph": {"iterations_per_replay": n_it, "bytes_per_iteration": int(graph_bytes),
                                     "ms_per_iteration": round(iter_graph_ms, 4), "achieved_GBs": round(graph_gbs, 1),
                                     "frac": round(graph_gbs / HBM_PEAK_GBS, 4),
                                     "adapter": "state half (h x h) per iteration, embedding half once per replay"},
                           "bytes": int(graph_bytes), "ms": round(iter_graph_ms, 4), "achieved_GBs": round(graph_gbs, 1),
                           "frac": round(graph_gbs / HBM_PEAK_GBS, 4)},
    }


def cpu_baseline(model, n_iters, r, seconds=12.0):
    """The CPU oracle (a port of the reference's CPU path) on the host cores: recurrence iterations
    (at least n_iters, then on until `seconds` of CPU work are spent, at most 400) plus LM-head products
    at the nebel shape, bs=1, 512 cached positions, scaled to tokens/s as
    1 / ((r + 1) * t_iteration + t_head) -- the 4 prelude/coda blocks cost one iteration.
    The only part of this file that touches the oracle."""
    import torch
    from oracle import raven_oracle as O
    shape = O.RavenShape.nebel()
    T = 512
    w = {}
    for name, p in model.state_dict().items():
        if name.startswith("transformer.core_block") or name.startswith("transformer.adapter") or name == "transformer.wte.weight":
            w[name] = p.detach().cpu()
    table = O.rope_table(shape.head_dim, shape.block_size, shape.rope_base).to(torch.bfloat16)
    g = torch.Generator().manual_seed(0)
    cache = O.DictCache()
    cache._seen_tokens = T
    kv = torch.randn(2, 1, shape.n_heads, T, shape.head_dim, generator=g).to(torch.bfloat16)
    x = O.initialize_state(torch.empty(1, 1, shape.n_embd), shape, 1.0, g).to(torch.bfloat16)
    emb = torch.randn(1, 1, shape.n_embd, generator=g).to(torch.bfloat16)
    n_threads = torch.get_num_threads()
    times = []
    while len(times) < n_iters + 1 or (sum(times[1:]) < seconds and len(times) < 401):  # first pass is warm-up
        for j in range(4):
            cache.key_cache[2 + j] = {p: kv[0, :, :, p] for p in range(T - 1)}
            cache.value_cache[2 + j] = {p: kv[1, :, :, p] for p in range(T - 1)}
        t0 = time.perf_counter()
        O.core_block_forward(x, emb, w, table[:, T - 1:T], cache, 1, shape)
        times.append(time.perf_counter() - t0)
    n_iters = len(times) - 1
    t_iter = sum(times[1:]) / max(1, n_iters)
    heads = []
    for _ in range(4):  # the first product is warm-up
        t0 = time.perf_counter()
        torch.nn.functional.linear(x, w["transformer.wte.weight"]).float()
        heads.append(time.perf_counter() - t0)
    t_head = sum(heads[1:]) / 3
    tok_s = 1.0 / ((r + 1) * t_iter + t_head)
    return {"value": round(tok_s, 5), "unit": "tokens/s", "cores": n_threads, "kind": "port",
            "sample": f"{n_iters} recurrence iterations ({sum(times[1:]):.1f} s, mean {t_iter * 1e3:.1f} ms) + 3 LM heads (mean {t_head * 1e3:.1f} ms) at nebel shape, "
                      f"bs=1, {T} cached positions, torch CPU bf16, {n_threads} threads of {os.cpu_count()} cpus; "
                      f"scaled to a token as ({r}+1) iterations + head"}


if __name__ == "__main__":
    main()
