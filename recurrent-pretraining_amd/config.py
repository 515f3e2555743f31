"""Model shape: the reference's RavenConfig (recpre/raven_config_minimal.py:7-99) as a transformers configuration
class, with the same field names, defaults, `attribute_map` and derived values, so a reference `config.json` loads
unchanged and `AutoConfig` resolves the model type `huginn_raven` to it (registration: raven_modeling_minimal.py:2312-2323).
Only the fields that shape inference are declared; the training-only keys of a reference file are kept as plain
attributes and written back on save."""

from __future__ import annotations

from math import sqrt

from transformers import PretrainedConfig

_NOISE_TYPES = ("geom", "sqrt", "line", "chi", "fixed")  # RMM:818-833


class RavenConfig(PretrainedConfig):
    model_type = "huginn_raven"
    keys_to_ignore_at_inference = [""]
    attribute_map = {"num_attention_heads": "n_heads", "hidden_size": "n_embd", "num_hidden_layers": "n_layers"}

    n_embd: int = 5280
    n_heads: int = 55
    n_layers: int = 8  # prelude + recurrent block + coda
    block_size: int = 4096
    vocab_size: int = 65536
    padding_multiple: int = 4096
    tie_embeddings: bool = True
    intermediate_size: int = 17920
    bias: bool = False
    norm_eps: float = 0.000001
    n_layers_in_recurrent_block: int = 4
    mean_recurrence: int = 32
    mean_backprop_depth: int = 8
    n_layers_in_prelude: int = 2
    n_layers_in_coda: int = 2
    qk_bias: bool = True
    rope_base: float = 50_000
    test_time_noise: float = 0
    test_time_noise_type: str = "fixed"

    def __post_init__(self, **kwargs):
        for alias, field in self.attribute_map.items():  # a file may name a field by its transformers-wide alias
            if kwargs.get(alias) is not None:
                setattr(self, field, kwargs[alias])
        if self.test_time_noise_type not in _NOISE_TYPES:
            raise ValueError(f"unknown test_time_noise_type {self.test_time_noise_type!r}")
        if self.test_time_noise < 0:
            raise ValueError("test_time_noise must not be negative")
        if self.bias:
            raise ValueError("bias=True is not supported: the reference model family has no Linear biases")
        if self.n_embd % self.n_heads:
            raise ValueError(f"n_embd {self.n_embd} is not divisible by n_heads {self.n_heads}")
        # derived values (raven_config_minimal.py:78-91); a file that stores them stores the same numbers
        for derived in ("padded_vocab_size", "num_key_value_heads", "num_attention_heads", "head_dim", "effective_expected_depth",
                        "init_values", "hidden_size", "num_hidden_layers"):
            kwargs.pop(derived, None)
        self.padded_vocab_size = self.vocab_size
        self.num_key_value_heads = self.n_heads
        self.head_dim = self.n_embd // self.n_heads
        self.effective_expected_depth = (self.n_layers_in_prelude + self.n_layers_in_coda
                                         + self.n_layers_in_recurrent_block * self.mean_recurrence)
        std = sqrt(2 / (5 * self.n_embd))
        self.init_values = {"std": std, "out_proj": std / sqrt(2 * self.effective_expected_depth), "embedding": std,
                            "embed_scale": sqrt(self.n_embd)}
        kwargs.pop("model_type", None)
        kwargs["tie_word_embeddings"] = self.tie_embeddings  # raven_config_minimal.py:93-99
        if self.dtype is None and kwargs.get("torch_dtype") is None:
            self.dtype = "bfloat16"  # the reference's default `torch_dtype`
        super().__post_init__(**kwargs)

    @classmethod
    def tiny(cls) -> "RavenConfig":
        """The CPU-runnable plumbing shape."""
        return cls(n_embd=256, n_heads=4, n_layers=4, n_layers_in_prelude=1, n_layers_in_recurrent_block=2,
                   n_layers_in_coda=1, intermediate_size=704, vocab_size=1024, mean_recurrence=4)
