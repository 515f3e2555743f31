"""Model shape, with the field names and derived values of the reference's RavenConfig
(recpre/raven_config_minimal.py:7-99).  A plain class: it does not need the transformers library,
but it reads the same JSON keys, so a reference `config.json` loads unchanged."""

from __future__ import annotations

import json
from math import sqrt


class RavenConfig:
    model_type = "huginn_raven"

    def __init__(
        self,
        n_embd: int = 5280,
        n_heads: int = 55,
        n_layers: int = 8,
        block_size: int = 4096,
        vocab_size: int = 65536,
        padding_multiple: int = 4096,
        tie_embeddings: bool = True,
        intermediate_size: int = 17920,
        bias: bool = False,
        norm_eps: float = 0.000001,
        n_layers_in_recurrent_block: int = 4,
        mean_recurrence: int = 32,
        mean_backprop_depth: int = 8,
        n_layers_in_prelude: int = 2,
        n_layers_in_coda: int = 2,
        qk_bias: bool = True,
        rope_base: float = 50_000,
        torch_dtype: str = "bfloat16",
        test_time_noise: float = 0,
        test_time_noise_type: str = "fixed",
        **kwargs,
    ):
        if test_time_noise_type not in ("geom", "sqrt", "line", "chi", "fixed"):  # RMM:818-833
            raise ValueError(f"unknown test_time_noise_type {test_time_noise_type!r}")
        if test_time_noise < 0:
            raise ValueError("test_time_noise must not be negative")
        if bias:
            raise ValueError("bias=True is not supported: the reference model family has no Linear biases")
        self.n_embd = n_embd
        self.n_heads = n_heads
        self.n_layers = n_layers
        self.block_size = block_size
        self.vocab_size = self.padded_vocab_size = vocab_size
        self.padding_multiple = padding_multiple
        self.tie_embeddings = tie_embeddings
        self.intermediate_size = intermediate_size
        self.bias = bias
        self.norm_eps = norm_eps
        self.n_layers_in_recurrent_block = n_layers_in_recurrent_block
        self.mean_recurrence = mean_recurrence
        self.mean_backprop_depth = mean_backprop_depth
        self.n_layers_in_prelude = n_layers_in_prelude
        self.n_layers_in_coda = n_layers_in_coda
        self.qk_bias = qk_bias
        self.rope_base = rope_base
        self.torch_dtype = torch_dtype
        self.test_time_noise = test_time_noise
        self.test_time_noise_type = test_time_noise_type
        self.extra = dict(kwargs)  # keys of the reference config that only matter for training
        # derived (raven_config_minimal.py:78-91)
        if n_embd % n_heads:
            raise ValueError(f"n_embd {n_embd} is not divisible by n_heads {n_heads}")
        self.num_key_value_heads = n_heads
        self.num_attention_heads = n_heads
        self.head_dim = n_embd // n_heads
        self.effective_expected_depth = n_layers_in_prelude + n_layers_in_coda + n_layers_in_recurrent_block * mean_recurrence
        self.init_values = {
            "std": sqrt(2 / (5 * n_embd)),
            "out_proj": sqrt(2 / (5 * n_embd)) / sqrt(2 * self.effective_expected_depth),
            "embedding": sqrt(2 / (5 * n_embd)),
            "embed_scale": sqrt(n_embd),
        }

    # names the transformers library uses for the same fields (raven_config_minimal.py:10)
    @property
    def hidden_size(self):
        return self.n_embd

    @property
    def num_hidden_layers(self):
        return self.n_layers

    @classmethod
    def from_json_file(cls, path: str) -> "RavenConfig":
        with open(path) as f:
            return cls(**json.load(f))

    @classmethod
    def tiny(cls) -> "RavenConfig":
        """The CPU-runnable plumbing shape."""
        return cls(n_embd=256, n_heads=4, n_layers=4, n_layers_in_prelude=1, n_layers_in_recurrent_block=2,
                   n_layers_in_coda=1, intermediate_size=704, vocab_size=1024, mean_recurrence=4)

    def to_dict(self) -> dict:
        keys = ("n_embd", "n_heads", "n_layers", "block_size", "vocab_size", "padding_multiple", "tie_embeddings",
                "intermediate_size", "bias", "norm_eps", "n_layers_in_recurrent_block", "mean_recurrence",
                "mean_backprop_depth", "n_layers_in_prelude", "n_layers_in_coda", "qk_bias", "rope_base", "torch_dtype",
                "test_time_noise", "test_time_noise_type")
        return {**self.extra, **{k: getattr(self, k) for k in keys}, "model_type": self.model_type}
