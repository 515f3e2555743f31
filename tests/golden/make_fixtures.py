"""Writes the fixtures of this directory.  Run from the repository root: python tests/golden/make_fixtures.py

The reference (seal-rg/recurrent-pretraining) ships no test vectors for the decode path; the only exact numbers it
publishes are the KV-cache sizes printed in examples/inference_demo.ipynb (cells at lines 252, 373, 491).  Those go into
reference_known_answers.json as they stand.  Everything else here is produced by this repository's CPU oracle
(oracle/raven_oracle.py, pinned by tests/test_oracle_pins.py) on seeded inputs, so that
  * a change of the oracle's arithmetic shows up as a changed fixture (tests/test_host_cpu.py compares), and
  * the GPU path can be checked against stored values without running the oracle (tests/test_gpu_model.py).
Nothing of the reference is imported or executed."""

import json
import os
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import raven_oracle as O  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def state_fn(s):
    return lambda call, shape: O.initialize_state(torch.empty(shape), s, 1.0, torch.Generator().manual_seed(7000 + call))


def main():
    torch.set_num_threads(4)
    s = O.RavenShape.tiny()
    w = O.make_weights(s, seed=0, dtype=torch.float32)
    ids = torch.randint(0, s.vocab_size, (2, 6), generator=torch.Generator().manual_seed(11))
    states = O.initialize_state(torch.empty(2, 6, s.n_embd), s, 1.0, torch.Generator().manual_seed(12))
    out = O.forward(w, s, input_ids=ids, input_states=states)
    greedy = O.greedy_generate(w, s, ids, 16, state_fn=state_fn(s))
    rec = {}
    adaptive, steps = O.generate_with_adaptive_compute(w, s, ids, 6, criterion="kl", exit_threshold=5e-3, num_steps=8,
                                                       state_fn=state_fn(s), cache_lookup_strategy="latest-m4", record=rec)
    spec = O.generate_speculative(w, s, ids[:1], 10, draft_steps=1, lookahead_for_draft=3, num_steps=4, init_scale=0.0)
    fx = {
        "config": "RavenShape.tiny(): h=256, 4 heads x 64, I=704, V=1024, 1 prelude / 2 core / 1 coda blocks, r=4; fp32; "
                  "weights make_weights(seed=0); prompt randint seed 11; states initialize_state seed 12 / 7000 + call",
        "prompt": ids.tolist(),
        "forward_last_logits_first8": [[round(float(v), 6) for v in row] for row in out.logits[:, -1, :8]],
        "forward_last_argmax": out.logits[:, -1].argmax(-1).tolist(),
        "forward_latent_l2": [round(float(v), 5) for v in out.latent_states[:, -1].norm(dim=-1)],
        "greedy_16_tokens": greedy[:, 6:].tolist(),
        "adaptive_kl_5e-3_tokens": adaptive[:, 6:].tolist(),
        "adaptive_kl_5e-3_compute_steps": steps,
        "speculative_draft1_look3_tokens": spec[:, 6:].tolist(),
    }
    with open(os.path.join(HERE, "tiny_fp32_oracle.json"), "w") as f:
        json.dump(fx, f, indent=1)
    ka = {
        "source": "seal-rg/recurrent-pretraining examples/inference_demo.ipynb (printed outputs of get_memory_usage())",
        "shape": "huginn-0125 / nebel-raven-3.5b: 55 heads x 96, bf16, 2 prelude + 4 core x 32 recurrences + 2 coda steps",
        "cases": [
            {"line": 252, "strategy": "full", "tokens": 366, "MB": 973.0810546875},
            {"line": 373, "strategy": "latest-m4-compress-s16", "tokens": 366, "MB": 147.4365234375},
            {"line": 491, "strategy": "static cache, max_length 1024, 132 steps, batch 1", "MB": 2722.5},
        ],
    }
    with open(os.path.join(HERE, "reference_known_answers.json"), "w") as f:
        json.dump(ka, f, indent=1)
    print("wrote", os.listdir(HERE))


if __name__ == "__main__":
    main()
