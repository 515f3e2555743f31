"""Host side of the MI355X recurrent-core decode path: a model class with the surface of the
reference's RavenForCausalLM (recpre/raven_modeling_minimal.py, "RMM": forward 638-724,
iterate_forward 726-762, core_block_forward 764-781, iterate_one_step 841-868, predict_from_latents
870-900, embed_inputs 902-934, generate_minimal 1165-1232) whose arithmetic runs in the HIP kernels
of libraven_hip.so.  torch.nn modules are used only as named parameter containers, so a reference
state dict loads with `load_state_dict` unchanged.  The class is a transformers `PreTrainedModel` with
`GenerationMixin` (RMM:36-112, 326), registered for `AutoConfig` / `AutoModel` / `AutoModelForCausalLM` under
the model type `huginn_raven` (RMM:2312-2323): a generate() call with none of the reference's own loop
keywords runs transformers' generation loop over this forward, as in the reference (RMM:1112-1127).

What differs from the reference on purpose:
  * token rows are processed as [B*S, h]; K/V live in one contiguous step-indexed buffer;
  * positions are one 1-D list shared by the batch, as in the reference (RMM:660-665); when they are not the tokens'
    cache indices the call rotates with a table gathered for it;
  * `attention_mask` is accepted and ignored, as in the reference (RMM:676);
  * only inference: no autograd, no labels-driven backward (a loss value is still returned).
"""

from __future__ import annotations

import math
import weakref
from dataclasses import dataclass
from typing import Any, Callable, Optional, Union

import torch
from transformers import AutoConfig, AutoModel, AutoModelForCausalLM, GenerationMixin, PreTrainedModel
from transformers.utils import ModelOutput

from . import hip
from .cache import HuginnDynamicCache, HuginnStaticCache, remap_step
from .config import RavenConfig


@dataclass
class CausalLMOutputRecurrentLatents(ModelOutput):  # RMM:113-123
    loss: Optional[torch.Tensor] = None
    log_ppl: Optional[torch.Tensor] = None
    logits: Optional[torch.Tensor] = None
    past_key_values: Optional[HuginnDynamicCache] = None
    latent_states: Optional[torch.Tensor] = None
    hidden_states: Optional[torch.Tensor] = None
    attention_maps: Optional[dict] = None
    stats: Optional[dict] = None


@dataclass
class GenerationSettings:
    """The fields of transformers.GenerationConfig that the generate loops read."""
    max_length: int = 4096
    max_new_tokens: Optional[int] = None
    do_sample: bool = False
    temperature: Optional[float] = None
    top_k: Optional[int] = None
    top_p: Optional[float] = None
    min_p: Optional[float] = None
    repetition_penalty: Optional[float] = None
    dry_multiplier: float = 0.0        # > 0 selects the n-gram penalty instead (RMM:2003-2046)
    dry_base: float = 1.75
    dry_allowed_length: int = 2
    eos_token_id: Any = None
    return_dict_in_generate: bool = False


@dataclass
class GenerateOutput:
    sequences: torch.Tensor
    past_key_values: Optional[HuginnDynamicCache] = None
    scores: Optional[dict] = None


# ------------------------------------------------------------------------------------------------
# parameter containers with the reference's module/parameter names (RMM:129-145, 439-452, 496-503, 512-523)
# ------------------------------------------------------------------------------------------------
class RMSNorm(torch.nn.Module):
    def __init__(self, dim: int, eps: float):
        super().__init__()
        self.eps = eps
        self.weight = torch.nn.Parameter(torch.ones(dim), requires_grad=False)


def _linear(n_in: int, n_out: int) -> torch.nn.Linear:
    lin = torch.nn.Linear(n_in, n_out, bias=False)
    lin.weight.requires_grad_(False)
    return lin


class CausalSelfAttention(torch.nn.Module):
    def __init__(self, cfg: RavenConfig):
        super().__init__()
        self.Wqkv = _linear(cfg.n_embd, 3 * cfg.n_embd)
        if cfg.qk_bias:
            self.qk_bias = torch.nn.Parameter(torch.zeros(2, 1, cfg.n_heads, cfg.head_dim), requires_grad=False)
        self.proj = _linear(cfg.n_embd, cfg.n_embd)


class GatedMLP(torch.nn.Module):
    def __init__(self, cfg: RavenConfig):
        super().__init__()
        self.fc = _linear(cfg.n_embd, 2 * cfg.intermediate_size)
        self.proj = _linear(cfg.intermediate_size, cfg.n_embd)


class SandwichBlock(torch.nn.Module):
    def __init__(self, cfg: RavenConfig, layer_id: int):
        super().__init__()
        self.norm_1 = RMSNorm(cfg.n_embd, cfg.norm_eps)
        self.attn = CausalSelfAttention(cfg)
        self.norm_2 = RMSNorm(cfg.n_embd, cfg.norm_eps)
        self.mlp = GatedMLP(cfg)
        self.norm_3 = RMSNorm(cfg.n_embd, cfg.norm_eps)
        self.norm_4 = RMSNorm(cfg.n_embd, cfg.norm_eps)
        self.layer_id = layer_id

    def native(self) -> hip.BlockWeights:
        a, m = self.attn, self.mlp
        bias = a.qk_bias if hasattr(a, "qk_bias") else None
        return hip.make_block_weights(self.norm_1.weight, self.norm_2.weight, self.norm_3.weight, self.norm_4.weight,
                                      a.Wqkv.weight, bias, a.proj.weight, m.fc.weight, m.proj.weight)


class _PackedWeights:
    """Line-aligned copies (hip.register_packed_weight) of the bf16 matrices whose rows are not whole 128-byte lines, read by
    the tiled GEMM in place of the originals for products over 33 and more token rows.  A copy belongs to a weight tensor's
    address and in-place version; `ensure` makes the copies again when either has changed (load_state_dict, .to()), `drop`
    unregisters them (also when the model is collected: the library's table is keyed by address)."""

    def __init__(self):
        self.key = None
        self.ptr_owner = []   # (weight tensor, packed buffer): both kept alive while registered

    def ensure(self, mats) -> None:
        mats = [w for w in mats if w.is_cuda and w.dtype == torch.bfloat16 and (w.shape[1] * 2) % 128 != 0 and w.shape[1] % 8 == 0]
        key = tuple((w.data_ptr(), w._version) for w in mats)
        if key == self.key:
            return
        # matrices that only changed in place keep their copy's buffer (a captured graph may hold its address)
        old = {(w.data_ptr(), tuple(w.shape)): buf for w, buf in self.ptr_owner}
        keep = {(w.data_ptr(), tuple(w.shape)) for w in mats}
        for w, _ in self.ptr_owner:
            if (w.data_ptr(), tuple(w.shape)) not in keep:
                hip.unregister_packed_weight(w)
        self.ptr_owner = [(w.detach(), hip.register_packed_weight(w.detach(), out=old.get((w.data_ptr(), tuple(w.shape))))) for w in mats]
        self.key = key

    def drop(self) -> None:
        for w, _ in self.ptr_owner:
            hip.unregister_packed_weight(w)
        self.ptr_owner = []
        self.key = None


def precompute_freqs_cis(dim: int, end: int, theta: float) -> torch.Tensor:
    """(cos, sin) table [1, end, 1, dim/2, 2] in fp32 (RMM:2076-2081)."""
    # always evaluated on the CPU, so the table does not depend on where the model lives
    inv = 1.0 / (theta ** (torch.arange(0, dim, 2, dtype=torch.float32, device="cpu") / dim))
    ang = torch.outer(torch.arange(end, dtype=torch.float32, device="cpu"), inv).float()
    return torch.stack([ang.cos()[None, :, None, :], ang.sin()[None, :, None, :]], dim=4)


def _as_int(v) -> int:
    return int(v.item()) if isinstance(v, torch.Tensor) else int(v)


class RavenPreTrainedModel(PreTrainedModel):
    """What transformers needs to know about the model family (RMM:36-112): the configuration class, the tied head, and
    the reference's weight initialisation for a model built from a configuration alone."""
    config_class = RavenConfig
    base_model_prefix = "model"
    supports_gradient_checkpointing = False  # inference only
    _no_split_modules = ["SandwichBlock"]
    _skip_keys_device_placement = ["past_key_values"]
    _tied_weights_keys = {"lm_head.weight": "transformer.wte.weight"}
    _supports_flash_attn = True
    _supports_sdpa = True
    _supports_attention_backend = True
    _tp_plan = {}

    @property
    def emb_scale(self) -> float:  # RMM:50-52
        return self.config.init_values["embed_scale"]

    @torch.no_grad()
    def _init_weights(self, module) -> None:
        """RMM:57-110 ("takase" scheme): truncated normals at +-3 std; Q, K, V and the two halves of fc drawn apart;
        output projections scaled down by the expected depth; norm weights one."""
        iv = self.config.init_values

        def normal(t, std):
            return torch.nn.init.trunc_normal_(t, mean=0.0, std=std, a=-3 * std, b=3 * std)

        names = getattr(self, "_module_names", None)
        if names is None:
            names = self._module_names = {id(m): n for n, m in self.named_modules()}
        name = names.get(id(module), "")
        if isinstance(module, RMSNorm):
            torch.nn.init.ones_(module.weight)
        elif isinstance(module, torch.nn.Embedding):
            normal(module.weight, iv["embedding"])
        elif isinstance(module, torch.nn.Linear):  # transformers visits the modules that own parameters
            if name.endswith("Wqkv"):
                for part in module.weight.split(self.config.n_embd, dim=0):  # n_kv_heads == n_heads: three h x h pieces
                    normal(part, iv["std"])
            elif name.endswith("mlp.fc"):
                gate, up = module.weight.chunk(2, dim=0)
                normal(gate, iv["std"])
                normal(up, iv["out_proj"])
            elif name.endswith("mlp.proj") or name.endswith("attn.proj"):
                normal(module.weight, iv["out_proj"])
            elif name.endswith("adapter") or (name == "lm_head" and not self.config.tie_embeddings):
                normal(module.weight, iv["std"])


class RavenForCausalLM(RavenPreTrainedModel, GenerationMixin):
    def __init__(self, config: RavenConfig, device: Union[str, torch.device, None] = None, dtype: Optional[torch.dtype] = None):
        """`device` None: wherever torch currently creates tensors (a `with torch.device(...)` block, transformers'
        loaders), else the GPU when there is one.  The parameters may live on the CPU; the forward needs them on the GPU."""
        super().__init__(config)
        if device is None:
            device = torch.get_default_device()
            if device.type == "cpu" and torch.cuda.is_available():
                device = torch.device("cuda")
        dtype = dtype if dtype is not None else (config.dtype if isinstance(config.dtype, torch.dtype) else torch.bfloat16)
        with torch.device(device):
            prelude = torch.nn.ModuleList(SandwichBlock(config, i) for i in range(config.n_layers_in_prelude))
            adapter = _linear(2 * config.n_embd, config.n_embd)
            core = torch.nn.ModuleList(SandwichBlock(config, i + config.n_layers_in_prelude)
                                       for i in range(config.n_layers_in_recurrent_block))
            o = config.n_layers_in_prelude + config.n_layers_in_recurrent_block * config.mean_recurrence
            coda = torch.nn.ModuleList(SandwichBlock(config, i + o) for i in range(config.n_layers_in_coda))
            wte = torch.nn.Embedding(config.padded_vocab_size, config.n_embd)
            wte.weight.requires_grad_(False)
            self.transformer = torch.nn.ModuleDict(dict(wte=wte, prelude=prelude, adapter=adapter, core_block=core,
                                                        coda=coda, ln_f=RMSNorm(config.n_embd, config.norm_eps)))
            self.lm_head = _linear(config.n_embd, config.padded_vocab_size)
            if config.tie_embeddings:
                self.lm_head.weight = self.transformer.wte.weight
            table = precompute_freqs_cis(config.head_dim, config.block_size, config.rope_base)
            self.register_buffer("freqs_cis", table.to(device), persistent=True)
        self.to(dtype)  # casts the RoPE table too, as nn.Module.to does for the reference (RMM:577)
        self.post_init()
        self.noise_source = None  # test-time noise draws: an object with normal(x) and uniform(x); None = torch's generator
        self._native_key = None
        self._native: dict = {}
        self._rope_override: Optional[torch.Tensor] = None  # a forward with positions that are not the cache's (see _rope_table_for)
        self._rope_memo = None                               # the last such table and what it was built for
        self._scratch: dict = {}
        self._packed = _PackedWeights()                      # line-aligned copies of weight matrices for prompt chunks
        self.pack_chunk_weights = True                       # False: chunks read the matrices as they are (no copies are made)
        self._packed_finalizer = weakref.finalize(self, self._packed.drop)
        self._packed_owner = id(self)
        self.eval()

    # ---- small helpers -------------------------------------------------------------------------
    @property
    def dtype(self) -> torch.dtype:
        return self.transformer.wte.weight.dtype

    @property
    def device(self) -> torch.device:
        return self.transformer.wte.weight.device

    def get_input_embeddings(self):
        return self.transformer.wte

    def get_output_embeddings(self):
        return self.lm_head

    def synthetic_weight_order(self) -> list:
        """Tensor names in the order the synthetic draw visits them: embedding, prelude blocks, adapter,
        core blocks, coda blocks, ln_f; inside a block norm_1, Wqkv, qk_bias, proj, norm_2, fc, mlp.proj,
        norm_3, norm_4."""
        cfg = self.config
        per_block = ["norm_1.weight", "attn.Wqkv.weight"] + (["attn.qk_bias"] if cfg.qk_bias else []) + [
            "attn.proj.weight", "norm_2.weight", "mlp.fc.weight", "mlp.proj.weight", "norm_3.weight", "norm_4.weight"]
        names = ["transformer.wte.weight"]
        for group, n in (("prelude", cfg.n_layers_in_prelude), ("adapter", 0), ("core_block", cfg.n_layers_in_recurrent_block),
                         ("coda", cfg.n_layers_in_coda)):
            if group == "adapter":
                names.append("transformer.adapter.weight")
            names += [f"transformer.{group}.{i}.{k}" for i in range(n) for k in per_block]
        names.append("transformer.ln_f.weight")
        if not cfg.tie_embeddings:
            names.append("lm_head.weight")
        return names

    @torch.no_grad()
    def init_weights(self, seed: Optional[int] = None, std: float = 0.02) -> None:
        """With a seed, synthetic weights: every tensor ~ N(0, std) (norm weights ~ N(1, std)), drawn on the CPU in
        synthetic_weight_order() from one seeded generator and cast, so that any host reproduces them.  Without one,
        what transformers calls at the end of construction: the reference's initialisation (_init_weights) and the tie."""
        if seed is None:
            return super().init_weights()
        g = torch.Generator(device="cpu").manual_seed(seed)
        sd = self.state_dict()
        for name in self.synthetic_weight_order():
            p = sd[name]
            mean = 1.0 if (name.endswith("weight") and p.dim() == 1) else 0.0
            p.copy_(torch.empty(p.shape, dtype=torch.float32).normal_(mean, std, generator=g).to(p.dtype))

    # ---- checkpoints -----------------------------------------------------------------------------
    _LOADER_KWARGS = ("trust_remote_code", "revision", "cache_dir", "token", "local_files_only", "force_download", "proxies",
                      "subfolder", "use_safetensors", "low_cpu_mem_usage", "attn_implementation", "code_revision", "adapter_kwargs",
                      "weights_only", "_from_auto", "_commit_hash", "use_auth_token", "resume_download", "state_dict", "variant")

    @classmethod
    def from_pretrained(cls, path: str, *model_args, device: Union[str, torch.device, None] = None,
                        dtype: Optional[torch.dtype] = None, config: Optional[RavenConfig] = None,
                        **kwargs) -> "RavenForCausalLM":
        """Builds the model from a LOCAL directory laid out like the reference's published checkpoints (what
        `AutoModelForCausalLM.from_pretrained(..., trust_remote_code=True)` reads for raven_modeling_minimal.py:2312-2323):
        `config.json` plus `model.safetensors`, or sharded `model-XXXXX-of-YYYYY.safetensors` with
        `model.safetensors.index.json`, or `pytorch_model.bin` (read with weights_only=True).  Nothing is downloaded.
        The parameter names are the reference's, so the tensors load unchanged; a tied head may be absent from the file.
        Replaces transformers' loader (one shard in host memory at a time, straight into the parameters) and takes its
        call shape: `config=` from an Auto class, `torch_dtype` / `dtype`, `device_map` as one device; the other loader
        keywords are accepted and have nothing to act on; any remaining keyword overrides a configuration field."""
        import json
        import os
        if dtype is None:
            dtype = kwargs.pop("torch_dtype", None)
        else:
            kwargs.pop("torch_dtype", None)
        if isinstance(dtype, str):
            dtype = None if dtype == "auto" else getattr(torch, dtype)
        device_map = kwargs.pop("device_map", None)
        if device is None and device_map is not None:
            if isinstance(device_map, dict):
                places = set(device_map.values())
                if len(places) != 1:
                    raise ValueError("the model lives on one device: device_map must name exactly one")
                device_map = places.pop()
            device = "cuda" if device_map == "auto" else device_map
        for k in cls._LOADER_KWARGS:
            kwargs.pop(k, None)
        path = str(path)
        if not os.path.isdir(path):
            raise FileNotFoundError(f"{path} is not a local directory (nothing is downloaded)")
        with open(os.path.join(path, "config.json")) as f:
            cfg_dict = json.load(f)
        if config is not None:
            cfg_dict = config.to_dict()
        cfg_dict.update(kwargs)
        config = RavenConfig(**cfg_dict)
        model = cls(config, device=device, dtype=dtype)
        index = os.path.join(path, "model.safetensors.index.json")
        single = os.path.join(path, "model.safetensors")
        legacy = os.path.join(path, "pytorch_model.bin")
        if os.path.exists(index):
            with open(index) as f:
                shards = sorted(set(json.load(f)["weight_map"].values()))
            files = [os.path.join(path, s) for s in shards]
        elif os.path.exists(single):
            files = [single]
        elif os.path.exists(legacy):
            files = [legacy]
        else:
            raise FileNotFoundError(f"no model.safetensors(.index.json) or pytorch_model.bin under {path}")
        own = model.state_dict()
        seen, unexpected = set(), []
        for file in files:  # shard by shard: at most one shard is held besides the model
            if file.endswith(".safetensors"):
                from safetensors.torch import load_file
                part = load_file(file, device="cpu")
            else:
                part = torch.load(file, map_location="cpu", weights_only=True)
            for name, tensor in part.items():
                if name not in own:
                    unexpected.append(name)
                    continue
                if own[name].shape != tensor.shape:
                    raise ValueError(f"{name}: checkpoint shape {tuple(tensor.shape)} != model shape {tuple(own[name].shape)}")
                own[name].copy_(tensor)
                seen.add(name)
            del part
        optional = {"freqs_cis"} | ({"lm_head.weight", "transformer.wte.weight"} if config.tie_embeddings else set())
        missing = [n for n in own if n not in seen and n not in optional]
        if config.tie_embeddings and not ({"lm_head.weight", "transformer.wte.weight"} & seen):
            missing.append("transformer.wte.weight")
        if missing or unexpected:
            raise KeyError(f"checkpoint does not match the model: missing {missing[:8]}, unexpected {unexpected[:8]}")
        model._native_key = None
        return model

    def save_pretrained(self, path: str, max_shard_bytes: int = 5 * 2 ** 30, **unused) -> None:
        """Writes `config.json` and safetensors shards (with an index when there are several) that from_pretrained and
        the reference's loader read.  The tied head is stored once, under the embedding's name."""
        import json
        import os
        from safetensors.torch import save_file
        path = str(path)
        os.makedirs(path, exist_ok=True)
        cfg = self.config.to_dict()
        cfg.update(architectures=["RavenForCausalLM"], torch_dtype=str(self.dtype).replace("torch.", ""))
        cfg["dtype"] = cfg["torch_dtype"]
        with open(os.path.join(path, "config.json"), "w") as f:
            json.dump(cfg, f, indent=1, sort_keys=True)
        sd = {k: v.detach().to("cpu").contiguous() for k, v in self.state_dict().items()
              if not (self.config.tie_embeddings and k == "lm_head.weight")}
        shards, cur, size = [], {}, 0
        for name, t in sd.items():
            nbytes = t.numel() * t.element_size()
            if cur and size + nbytes > max_shard_bytes:
                shards.append(cur)
                cur, size = {}, 0
            cur[name] = t
            size += nbytes
        shards.append(cur)
        if len(shards) == 1:
            save_file(shards[0], os.path.join(path, "model.safetensors"), metadata={"format": "pt"})
            return
        weight_map = {}
        for i, part in enumerate(shards):
            fname = f"model-{i + 1:05d}-of-{len(shards):05d}.safetensors"
            save_file(part, os.path.join(path, fname), metadata={"format": "pt"})
            weight_map.update({k: fname for k in part})
        with open(os.path.join(path, "model.safetensors.index.json"), "w") as f:
            json.dump({"metadata": {"total_size": sum(t.numel() * t.element_size() for t in sd.values())}, "weight_map": weight_map}, f,
                      indent=1)

    def _natives(self) -> dict:
        """ctypes views of the weights; rebuilt when a parameter's storage has moved."""
        key = (self.transformer.wte.weight.data_ptr(), self.transformer.adapter.weight.data_ptr(),
               self.freqs_cis.data_ptr(), self.transformer.ln_f.weight.data_ptr(), self.dtype)
        if key != self._native_key:
            cfg, t = self.config, self.transformer
            core = (hip.BlockWeights * len(t.core_block))(*[b.native() for b in t.core_block])
            self._native = {
                "dims": hip.make_dims(cfg.n_embd, cfg.n_heads, cfg.intermediate_size, cfg.norm_eps, self.dtype),
                "prelude": [b.native() for b in t.prelude],
                "core": core,
                "coda": [b.native() for b in t.coda],
                "freqs": self.freqs_cis.float().reshape(cfg.block_size, cfg.head_dim // 2, 2).contiguous(),
            }
            self._native_key = key
            self._scratch.clear()
        return self._native

    def _workspace(self, M: int) -> torch.Tensor:
        """Scratch for a block over M token rows; every block call fetches it, so this is also where a call over 17 rows or
        more (decode steps of 17..32 sequences read Wqkv and mlp.fc through them, chunks of 33 rows and more all three matrices)
        makes sure that the line-aligned weight copies are current."""
        if M >= 17 and self.dtype == torch.bfloat16 and self.pack_chunk_weights:
            self.pack_weights()
        ws = self._scratch.get(("ws", M))
        if ws is None:
            ws = hip.block_workspace(self._natives()["dims"], M, self.device)
            self._scratch[("ws", M)] = ws
        return ws

    def _scratch_cache(self, B: int, S: int) -> HuginnDynamicCache:
        """A one-slot cache for forwards without past_key_values: every block appends its S new
        keys to it and attends causally, which is what the reference does with no cache."""
        key = ("nocache", B)
        c = self._scratch.get(key)
        cfg = self.config
        if c is None or c.t_max < S:
            c = HuginnDynamicCache()
            c.ensure(1, 0, B, cfg.n_heads, cfg.head_dim, S, self.dtype, self.device)
            self._scratch[key] = c
        return c

    def _rope_positions(self, n_tokens: int, position_ids, cache_position) -> list:
        """The RoPE positions of this call's tokens, shared by the batch (RMM:660-665): `position_ids` squeezed to one
        dimension, else `cache_position`, else 0 .. S-1.  Any values inside the table are allowed; they only pick rows of
        the RoPE table, the cache index of a token is the number of tokens the cache has seen."""
        src = position_ids if position_ids is not None else cache_position
        if src is None:
            return list(range(n_tokens))
        if src.dim() == 2 and src.shape[0] > 1:  # one row per sequence, as transformers' generate() builds them
            if not bool((src == src[:1]).all()):
                raise ValueError("positions differ between the sequences of the batch: they are one list shared by the batch "
                                 "(a left-padded batch cannot be rotated row by row, RMM:660-665)")
            src = src[0]
        pos = [int(v) for v in src.reshape(-1).tolist()]
        if len(pos) != n_tokens:
            raise ValueError(f"{len(pos)} positions for {n_tokens} tokens: positions are one 1-D list shared by the batch")
        if min(pos) < 0 or max(pos) >= self.config.block_size:
            raise IndexError(f"positions {min(pos)} .. {max(pos)} outside the RoPE table of {self.config.block_size} rows")
        return pos

    def _rope_table_for(self, rope_pos: list, cache_pos0: int) -> Optional[torch.Tensor]:
        """None when the tokens' RoPE positions are their cache positions (cache_pos0, cache_pos0 + 1, ...): the kernels
        then read the model's table.  Otherwise a table for this call whose rows cache_pos0 + i hold the model's rows
        rope_pos[i] (the kernels rotate the token at cache index p with row p)."""
        if all(p == cache_pos0 + i for i, p in enumerate(rope_pos)):
            return None
        full = self._natives()["freqs"]
        key = (cache_pos0, tuple(rope_pos), full.data_ptr())
        if self._rope_memo is not None and self._rope_memo[0] == key:   # a batch that stays out of step asks for the same table again
            return self._rope_memo[1]
        table = torch.zeros(cache_pos0 + len(rope_pos), full.shape[1], 2, dtype=full.dtype, device=full.device)
        table[cache_pos0:] = full[torch.as_tensor(rope_pos, device=full.device)]
        self._rope_memo = (key, table)
        return table

    def _freqs(self) -> torch.Tensor:
        return self._rope_override if self._rope_override is not None else self._natives()["freqs"]

    def _split_steps(self, num_steps) -> int:
        """Total recurrences (RMM:739-744; eval sampler RMM:799-802)."""
        if num_steps is None:
            return self.config.mean_recurrence
        if isinstance(num_steps, torch.Tensor) and num_steps.dim() == 0:
            return int(num_steps)
        if hasattr(num_steps, "__len__") and len(num_steps) > 1:
            return int(num_steps[0]) + int(num_steps[1])
        return int(num_steps)

    # ---- pieces of the forward --------------------------------------------------------------------
    def _run_block(self, which: str, i: int, step_idx: int, x: torch.Tensor, cache: HuginnDynamicCache, private: bool,
                   B: int, S: int, pos0: int, ln_f: bool = False) -> torch.Tensor:
        nat = self._natives()
        slot = 0 if private else cache.note_append(step_idx, S, pos0)
        kv = cache.native() if private else cache.native([step_idx], pos0)
        out = torch.empty_like(x)
        hip.sandwich_block(nat["dims"], nat[which][i], x, out, self._freqs(), kv, slot, B, S, pos0,
                           self._workspace(B * S), ln_f=self.transformer.ln_f.weight if ln_f else None)
        return out

    def _maybe_inject_noise(self, x: torch.Tensor, current_step: int, renorm: bool = True) -> torch.Tensor:
        """RMM:815-837: with test_time_noise set, the state is mixed with fresh Gaussian noise in front of every
        recurrence and passed through the last core block's norm_4 again.  The draws come from self.noise_source
        (`normal(x)`, `uniform(x)`) when that is set, otherwise from torch's generator of the device."""
        cfg = self.config
        if cfg.test_time_noise <= 0:
            return x
        n = cfg.test_time_noise * cfg.init_values["std"] * self.emb_scale
        src = self.noise_source
        kind = cfg.test_time_noise_type
        # The reference's expression mixes Python floats (taken as float32 operands by the elementwise kernels) with 0-dim
        # device tensors (converted to the state's dtype first, as ATen's GPU kernels do); every product, quotient and
        # sum is rounded to the state's dtype.
        f32 = lambda v: float(torch.tensor(v, dtype=torch.float32))
        as_state = lambda v: float(torch.tensor(v, dtype=torch.float32).to(x.dtype))
        d = 0.0
        if kind in ("geom", "sqrt"):  # n / (step + 1) or n / sqrt(step + 1): float32 0-dim tensors (RMM:819-823)
            d32 = f32(current_step + 1) if kind == "geom" else f32(math.sqrt(current_step + 1))
            keep, a, d = as_state(1.0 - f32(f32(n) / d32)), n, as_state(d32)
        elif kind == "line":          # RMM:825-826, a Python float
            c = max(n, (cfg.mean_recurrence - current_step) / cfg.mean_recurrence)
            keep, a = 1.0 - c, c
        elif kind == "chi":           # RMM:828-829: 2 * rand(1) * n, a tensor of the state's dtype
            u = src.uniform(x) if src is not None else torch.rand(1, device=x.device, dtype=x.dtype)
            c = as_state(as_state(2.0 * float(u)) * f32(n))
            keep, a = as_state(1.0 - c), c
        else:                         # "fixed", RMM:831
            keep, a = 1.0 - n, n
        noise = src.normal(x).to(device=x.device, dtype=x.dtype) if src is not None else torch.randn_like(x)
        x = hip.noise_mix(x, noise.reshape(x.shape).contiguous(), keep, a, d)
        if renorm:
            x = hip.rmsnorm_residual(x, self.transformer.core_block[-1].norm_4.weight, cfg.norm_eps)[0]
        return x

    def _run_core(self, x: torch.Tensor, embeds: torch.Tensor, first_step: int, cache: HuginnDynamicCache, private: bool,
                  B: int, S: int, pos0: int, ln_f: bool, current_step: int = 0) -> torch.Tensor:
        """One core_block_forward (RMM:764-781) on [B*S, h] rows."""
        nat, t = self._natives(), self.transformer
        x = self._maybe_inject_noise(x, current_step)
        n_core = len(t.core_block)
        slots = [0 if private else cache.note_append(first_step + j, S, pos0) for j in range(n_core)]
        # positions of earlier tokens that were computed with fewer recurrences are not cached at these steps:
        # the attention kernels then follow the cache's lookup strategy (one descriptor per launch)
        steps = [first_step + j for j in range(n_core)]
        gaps = [False] * n_core if private else [cache.has_gap(s_, pos0) for s_ in steps]
        uniform = all(g == gaps[0] for g in gaps)
        kv = cache.native() if private or not uniform else cache.native(steps, pos0)
        out = torch.empty_like(x)
        ws = self._workspace(B * S)
        lnw = t.ln_f.weight if ln_f else None
        if not private and uniform and n_core > 0 and all(slots[j] == slots[0] + j for j in range(n_core)):
            hip.core_iteration(nat["dims"], t.adapter.weight, nat["core"], x, embeds, out, self._freqs(), kv,
                               slots[0], B, S, pos0, ws, ln_f=lnw)
            return out
        cur = hip.linear(x, t.adapter.weight, x1=embeds, workspace=ws)  # the kernels raven_core_iteration would pick
        for j in range(n_core):
            last = j == n_core - 1
            nxt = out if last else torch.empty_like(x)
            kv_j = kv if uniform else cache.native([steps[j]], pos0)
            hip.sandwich_block(nat["dims"], nat["core"][j], cur, nxt, self._freqs(), kv_j, slots[j], B, S, pos0, ws,
                               ln_f=lnw if last else None)
            cur = nxt
        if n_core == 0:
            out = cur if lnw is None else hip.rmsnorm_residual(cur, lnw, self.config.norm_eps)[0]
        return out

    @torch.no_grad()
    def initialize_state(self, input_embeds: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
        """RMM:804-813, with torch's generator of the tensor's device."""
        x = torch.randn_like(input_embeds)
        std = self.config.init_values["std"] * scale
        if std > 0:
            torch.nn.init.trunc_normal_(x, mean=0.0, std=std, a=-3 * std, b=3 * std)
            if self.emb_scale != 1:
                x = x * self.emb_scale
        else:
            x.zero_()
        return x

    def _prepare_cache(self, past_key_values, use_cache: bool, B: int, S: int, r: int):
        """Returns (cache, private, cache_pos0) and reserves storage for this call's steps."""
        cfg = self.config
        if use_cache and past_key_values is None:
            past_key_values = HuginnDynamicCache()
        if past_key_values is None:
            return self._scratch_cache(B, S), True, 0
        if not isinstance(past_key_values, HuginnDynamicCache):
            raise TypeError("past_key_values must be this package's HuginnDynamicCache")
        cache = past_key_values
        pos0 = cache._seen_tokens
        n_pos = cfg.n_layers_in_prelude + cfg.n_layers_in_recurrent_block * r
        n_pos = max((remap_step(s, cache.lookup_strategy) for s in range(n_pos)), default=-1) + 1
        cache.ensure(max(n_pos, 1), cfg.n_layers_in_coda, B, cfg.n_heads, cfg.head_dim, pos0 + S, self.dtype, self.device)
        return cache, False, pos0

    # ---- reference surface -----------------------------------------------------------------------
    @torch.no_grad()
    def forward(
        self,
        input_ids: Optional[torch.Tensor] = None,
        input_embeds: Optional[torch.Tensor] = None,
        input_states: Optional[torch.Tensor] = None,
        attention_mask: Optional[torch.Tensor] = None,
        position_ids: Optional[torch.Tensor] = None,
        labels: Optional[torch.Tensor] = None,
        num_steps=None,
        past_key_values: Optional[HuginnDynamicCache] = None,
        output_details: dict = {"return_logits": True, "return_latents": True, "return_head": False, "return_stats": False},
        use_cache: bool = False,
        cache_position: Optional[torch.Tensor] = None,
        init_scale: float = 1.0,
        **kwargs,
    ) -> CausalLMOutputRecurrentLatents:
        cfg, t = self.config, self.transformer
        src = input_ids if input_embeds is None else input_embeds
        B, S = src.shape[0], src.shape[1]
        M, h = B * S, cfg.n_embd
        rope_pos = self._rope_positions(S, position_ids, cache_position)
        r = self._split_steps(num_steps)
        cache, private, pos0 = self._prepare_cache(past_key_values, use_cache, B, S, r)
        override = self._rope_table_for(rope_pos, pos0)
        if not private:
            cache._seen_tokens += S  # what the step-0 update does in the reference (RMM:188-189)
        self._rope_override = override
        try:
            return self._forward_rows(input_ids, input_embeds, input_states, labels, output_details, init_scale, cache, private, pos0,
                                      B, S, r)
        finally:
            self._rope_override = None

    def pack_weights(self) -> None:
        """Makes (or refreshes) the line-aligned copies of Wqkv, attn.proj and mlp.fc that products over 33 and more token rows
        read (bf16 models whose n_embd * 2 bytes is not a multiple of 128: n_embd = 5280).  Every block call over such a
        chunk calls this; call it by hand after changing a weight through `.data`, which leaves no trace a check could see."""
        if not self._packed_finalizer.alive or self._packed_owner != id(self):
            # a copy of a model (copy.deepcopy) starts without registrations of its own
            self._packed = _PackedWeights()
            self._packed_finalizer = weakref.finalize(self, self._packed.drop)
            self._packed_owner = id(self)
        t = self.transformer
        blocks = list(t.prelude) + list(t.core_block) + list(t.coda)
        self._packed.ensure([w for b in blocks for w in (b.attn.Wqkv.weight, b.attn.proj.weight, b.mlp.fc.weight)])

    def _forward_rows(self, input_ids, input_embeds, input_states, labels, output_details, init_scale, cache, private, pos0, B, S, r):
        cfg, t = self.config, self.transformer
        M, h = B * S, cfg.n_embd

        if input_embeds is None:
            x = hip.embed(t.wte.weight, input_ids.reshape(-1).to(torch.int64).contiguous(), self.emb_scale)
        else:
            x = (input_embeds.to(self.dtype) * self.emb_scale).reshape(M, h).contiguous()

        block_idx = -1
        for i in range(len(t.prelude)):
            block_idx += 1
            x = self._run_block("prelude", i, block_idx, x, cache, private, B, S, pos0)
        embeds = x

        if input_states is None:
            state = self.initialize_state(embeds, init_scale)
        else:
            state = input_states.to(self.dtype).reshape(M, h).clone()
        x = self._iterate(state, embeds, block_idx, cache, private, B, S, pos0, r)
        latents = x.view(B, S, h).clone()

        n_coda = len(t.coda)
        for i in range(n_coda):
            x = self._run_block("coda", i, -(i + 1), x, cache, private, B, S, pos0, ln_f=(i == n_coda - 1))
        if n_coda == 0:
            x = hip.rmsnorm_residual(x, t.ln_f.weight, cfg.norm_eps)[0]

        logits = hip.gemm(x, self.lm_head.weight, out_f32=True).view(B, S, -1)
        if labels is not None:
            loss = torch.nn.functional.cross_entropy(logits.view(-1, logits.shape[-1]), labels.view(-1), ignore_index=-100)
            log_ppl = loss.clone()
        else:
            loss, log_ppl = torch.as_tensor(0.0), torch.as_tensor(0.0)
        return CausalLMOutputRecurrentLatents(
            loss=loss, log_ppl=log_ppl,
            logits=logits if output_details.get("return_logits", True) else None,
            past_key_values=None if private else cache,
            hidden_states=x.view(B, S, h) if output_details.get("return_head", False) else None,
            latent_states=latents if output_details.get("return_latents", True) else None,
        )

    def _iterate(self, state, embeds, block_idx: int, cache, private, B, S, pos0, r: int) -> torch.Tensor:
        """The r-loop of iterate_forward plus its closing ln_f (RMM:751-762)."""
        n_core = len(self.transformer.core_block)
        x = state
        for it in range(r):
            x = self._run_core(x, embeds, block_idx + 1 + it * n_core, cache, private, B, S, pos0, ln_f=(it == r - 1), current_step=it)
        if r == 0:
            x = hip.rmsnorm_residual(x, self.transformer.ln_f.weight, self.config.norm_eps)[0]
        return x

    @torch.no_grad()
    def iterate_forward(self, input_embeds, input_states, freqs_cis=None, block_idx=None, mask=None, past_key_values=None,
                        num_steps=None, init_scale: float = 1.0):
        """RMM:726-762.  `freqs_cis` is not needed (positions follow from the cache) and is ignored.
        Returns (ln_f(x), n_no_grad, n_grad, None, block_idx)."""
        B, S, h = input_embeds.shape
        r = self._split_steps(num_steps)
        b0 = _as_int(block_idx) if block_idx is not None else len(self.transformer.prelude) - 1
        cache, private, pos0 = self._cache_for_piece(past_key_values, B, S, b0 + 1 + r * len(self.transformer.core_block))
        embeds = input_embeds.to(self.dtype).reshape(B * S, h).contiguous()
        state = (self.initialize_state(embeds, init_scale) if input_states is None
                 else input_states.to(self.dtype).reshape(B * S, h).clone())
        x = self._iterate(state, embeds, b0, cache, private, B, S, pos0, r)
        out_idx = torch.tensor(b0 + r * len(self.transformer.core_block), dtype=torch.long)
        return x.view(B, S, h), r, 0, None, out_idx

    def _cache_for_piece(self, past_key_values, B: int, S: int, n_pos_steps: int):
        """Cache handling for the per-piece entry points, which run after step 0 has already
        advanced the token count: the new tokens sit at _seen_tokens - S (RMM:194)."""
        cfg = self.config
        if past_key_values is None:
            return self._scratch_cache(B, S), True, 0
        cache = past_key_values
        pos0 = cache._seen_tokens - S
        if pos0 < 0:
            raise ValueError("the cache has seen fewer tokens than this call brings: run embed_inputs first")
        n_pos = max((remap_step(s, cache.lookup_strategy) for s in range(n_pos_steps)), default=-1) + 1
        cache.ensure(max(n_pos, 1), cfg.n_layers_in_coda, B, cfg.n_heads, cfg.head_dim, pos0 + S, self.dtype, self.device)
        return cache, False, pos0

    @torch.no_grad()
    def core_block_forward(self, x, input_embeds, freqs_cis=None, mask=None, past_key_values=None, block_idx=0,
                           current_step=0):
        """RMM:764-781: one recurrence; returns (x, block_idx + n_core)."""
        B, S, h = x.shape
        b0 = _as_int(block_idx)
        n_core = len(self.transformer.core_block)
        cache, private, pos0 = self._cache_for_piece(past_key_values, B, S, b0 + 1 + n_core)
        out = self._run_core(x.to(self.dtype).reshape(B * S, h).contiguous(),
                             input_embeds.to(self.dtype).reshape(B * S, h).contiguous(), b0 + 1, cache, private, B, S, pos0,
                             ln_f=False, current_step=_as_int(current_step))
        return out.view(B, S, h), torch.tensor(b0 + n_core, dtype=torch.long)

    @torch.no_grad()
    def iterate_one_step(self, input_embeds, input_states, position_ids=None, cache_position=None,
                         block_idx=torch.tensor(0, dtype=torch.long), attention_mask=None, past_key_values=None,
                         current_step: int = 0):
        """RMM:841-868."""
        x, block_idx = self.core_block_forward(input_states, input_embeds, None, attention_mask, past_key_values, block_idx,
                                               current_step)
        return x, block_idx, current_step + 1

    @torch.no_grad()
    def predict_from_latents(self, latents, attention_mask=None, position_ids=None, cache_position=None,
                             past_key_values=None):
        """RMM:870-900: ln_f, coda, ln_f, head."""
        cfg, t = self.config, self.transformer
        B, S, h = latents.shape
        cache, private, pos0 = self._cache_for_piece(past_key_values, B, S, 1)
        x = hip.rmsnorm_residual(latents.to(self.dtype).reshape(B * S, h).contiguous(), t.ln_f.weight, cfg.norm_eps)[0]
        n_coda = len(t.coda)
        for i in range(n_coda):
            x = self._run_block("coda", i, -(i + 1), x, cache, private, B, S, pos0, ln_f=(i == n_coda - 1))
        if n_coda == 0:
            x = hip.rmsnorm_residual(x, t.ln_f.weight, cfg.norm_eps)[0]
        logits = hip.gemm(x, self.lm_head.weight, out_f32=True).view(B, S, -1)
        return CausalLMOutputRecurrentLatents(loss=torch.as_tensor(0.0), log_ppl=torch.as_tensor(0.0), logits=logits,
                                              past_key_values=past_key_values, latent_states=x.view(B, S, h))

    @torch.no_grad()
    def embed_inputs(self, input_ids, attention_mask=None, position_ids=None, past_key_values=None, use_cache=False,
                     cache_position=None, **kwargs):
        """RMM:902-934: embedding times sqrt(h), then the prelude; returns (embeds, block_idx)."""
        cfg, t = self.config, self.transformer
        B, S = input_ids.shape
        rope_pos = self._rope_positions(S, position_ids, cache_position)
        cache, private, pos0 = self._prepare_cache(past_key_values, use_cache, B, S, 0)
        self._rope_override = self._rope_table_for(rope_pos, pos0)
        if not private:
            cache._seen_tokens += S
        try:
            x = hip.embed(t.wte.weight, input_ids.reshape(-1).to(torch.int64).contiguous(), self.emb_scale)
            block_idx = -1
            for i in range(len(t.prelude)):
                block_idx += 1
                x = self._run_block("prelude", i, block_idx, x, cache, private, B, S, pos0)
        finally:
            self._rope_override = None
        return x.view(B, S, cfg.n_embd), torch.tensor(block_idx, dtype=torch.long)

    # ---- generation --------------------------------------------------------------------------------
    @classmethod
    def _supports_default_dynamic_cache(cls) -> bool:
        """transformers' generate() must not build its own per-layer cache: the forward makes a HuginnDynamicCache."""
        return False

    def prepare_inputs_for_generation(self, input_ids, next_sequence_length=None, past_key_values=None, attention_mask=None,
                                      inputs_embeds=None, is_first_iteration=False, cache_position=None,
                                      cache_lookup_strategy: str = "full", **kwargs):
        """What transformers' generation loop calls before every forward (RMM:1066-1110).  It selects the tokens to feed:
        `input_ids[:, cache_position]` when the loop tracks cache positions (transformers 4.x, as in the reference), else
        the last `next_sequence_length` tokens (5.x), else all of them.  A cache of another class (the loop's own
        default) must be empty and is replaced by this package's, as the reference does; `attention_mask` is accepted
        and not forwarded (the forward ignores it, RMM:676)."""
        model_inputs = {}
        if past_key_values is not None and not isinstance(past_key_values, HuginnDynamicCache):
            if past_key_values.get_seq_length() != 0:
                raise ValueError("only an empty cache of another class can be replaced by a HuginnDynamicCache")
            if type(past_key_values).__name__ == "StaticCache":
                cfg = self.config
                past_key_values = HuginnStaticCache(
                    max_length=min(getattr(self.generation_config, "max_length", None) or cfg.block_size, cfg.block_size),
                    max_num_steps=4 + kwargs.get("num_steps", cfg.mean_recurrence) * 4, num_heads=cfg.num_key_value_heads,
                    hidden_dim=cfg.head_dim, batch_size=input_ids.shape[0], device=self.device, dtype=self.dtype,
                    lookup_strategy=cache_lookup_strategy)
            else:
                past_key_values = HuginnDynamicCache(cache_lookup_strategy)
        use_cache = kwargs.get("use_cache", True)
        model_inputs["past_key_values"] = past_key_values if use_cache else None
        if cache_position is not None:
            model_inputs["cache_position"] = cache_position
            input_ids = input_ids[:, cache_position]
        elif next_sequence_length is not None:
            input_ids = input_ids[:, -next_sequence_length:]
        model_inputs["input_ids"] = input_ids.clone(memory_format=torch.contiguous_format)
        position_ids = kwargs.pop("position_ids", None)
        if position_ids is not None and cache_position is None:
            model_inputs["position_ids"] = position_ids[..., -input_ids.shape[1]:].clone(memory_format=torch.contiguous_format)
        for key, value in kwargs.items():
            if key not in model_inputs and key not in ("labels", "next_sequence_length"):
                model_inputs[key] = value
        return model_inputs

    def _get_stops(self, generation_config, model_kwargs=None) -> set:
        stops = {65504, 65505, 65508}  # begin_text, end_text, end_turn (RMM:1929-1931)
        eos = getattr(generation_config, "eos_token_id", None)
        if eos is not None:
            try:
                stops.update(eos)
            except TypeError:
                stops.add(eos)
        return stops

    def _sample_next_token(self, next_token_logits: torch.Tensor, input_ids, generation_config) -> torch.Tensor:
        """RMM:1944-1989.  Greedy selection runs in the HIP argmax kernel."""
        gc = generation_config
        if getattr(gc, "repetition_penalty", None) is not None and gc.repetition_penalty != 1.0:
            next_token_logits = self._apply_repetition_penalty(next_token_logits, input_ids, gc)
        if not getattr(gc, "do_sample", False):
            return hip.argmax(next_token_logits.float().contiguous()).unsqueeze(-1)
        logits = next_token_logits.to(torch.float32)
        if gc.temperature:
            logits = logits / gc.temperature
        probs = torch.softmax(logits, dim=-1)
        if gc.top_k:
            kth = torch.topk(probs, gc.top_k, dim=-1).values[:, -1:]
            probs = torch.where(probs < kth, torch.zeros_like(probs), probs)
        if gc.top_p:
            sp, si = torch.sort(probs, descending=True, dim=-1)
            remove = torch.cumsum(sp, dim=-1) > gc.top_p
            remove[:, 0] = False
            mask = torch.zeros_like(probs, dtype=torch.bool).scatter(1, si, remove)
            probs = torch.where(mask, torch.zeros_like(probs), probs)
        if gc.min_p:
            probs = torch.where(probs < gc.min_p * probs.max(dim=-1, keepdim=True).values, torch.zeros_like(probs), probs)
        probs = probs / probs.sum(dim=-1, keepdim=True).clamp(min=1e-10)
        return torch.multinomial(probs, num_samples=1)

    def _default_max_length(self, gc) -> int:
        """`max_length` of the generation settings; transformers 5 leaves it unset by default, then the RoPE table's length."""
        for src in (gc, self.generation_config):
            if getattr(src, "max_length", None):
                return src.max_length
        return self.config.block_size

    def _generation_cache(self, model_kwargs: dict, cache_lookup_strategy: str, batch: int, max_length: Optional[int] = None):
        """The cache a generate loop works on (RMM:1146-1160): the caller's `past_key_values`, or a new one --
        HuginnStaticCache when `cache_implementation="static"` is asked for, else HuginnDynamicCache."""
        given = model_kwargs.get("past_key_values")
        if given is not None:
            return given
        if model_kwargs.get("cache_implementation", "dynamic") == "static":
            cfg = self.config
            length = max_length if max_length is not None else model_kwargs.get("max_length", self._default_max_length(None))
            steps = 4 + model_kwargs.get("num_steps", cfg.mean_recurrence) * 4
            return HuginnStaticCache(max_length=min(length, cfg.block_size), max_num_steps=steps, num_heads=cfg.num_key_value_heads,
                                     hidden_dim=cfg.head_dim, batch_size=batch, device=self.device, dtype=self.dtype,
                                     lookup_strategy=cache_lookup_strategy)
        return HuginnDynamicCache(cache_lookup_strategy, max_length=max_length)

    def _apply_repetition_penalty(self, original_logits, input_ids, generation_config, use_candidates: bool = False):
        """RMM:1991-2070; see sampling.apply_repetition_penalty."""
        from .sampling import apply_repetition_penalty
        return apply_repetition_penalty(original_logits, input_ids, generation_config, use_candidates)

    def get_stats(self, logits, x, latent_states, xk, input_embeds, num_steps_no_grad, num_steps_with_grad) -> dict:
        """RMM:1037-1049: entropy of the predictive distribution and the distance between two latent states."""
        probs = torch.softmax(logits.float(), dim=-1)
        residual_diff = (x - latent_states).norm(dim=-1)
        return {"entropy": torch.where(probs > 0, -probs * probs.log(), 0).sum(dim=-1), "residual_diff": residual_diff,
                "rel_residual": residual_diff / latent_states.norm(dim=-1), "num_steps_no_grad": num_steps_no_grad,
                "num_steps_with_grad": num_steps_with_grad}

    _MINIMAL_LOOP_KEYS = ("continuous_compute", "input_states_fn", "stop_tokens", "use_graph")

    @torch.no_grad()
    def generate(self, input_ids: Optional[torch.Tensor] = None, generation_config=None, **kwargs):
        """Dispatcher of RMM:1112-1127: `criterion` / `exit_threshold` / `exit_evaluator` select the adaptive-compute
        loop, `draft_steps` / `lookahead_for_draft` / `verification_threshold` the self-speculative one, `headway` /
        `state_noise_mixing` / `inner_recurrence` / `freeze_strategy` the diffusion-style one, `continuous_compute` (and
        this package's own `input_states_fn` / `stop_tokens` / `use_graph`, or a GenerationSettings) generate_minimal;
        every other call is transformers' GenerationMixin.generate over this model's forward."""
        if any(k in kwargs for k in ("criterion", "exit_threshold", "exit_evaluator")):
            return self.generate_with_adaptive_compute(input_ids, generation_config, **kwargs)
        if any(k in kwargs for k in ("draft_steps", "lookahead_for_draft", "verification_threshold")):
            return self.generate_speculative(input_ids, generation_config, **kwargs)
        if any(k in kwargs for k in ("headway", "state_noise_mixing", "inner_recurrence", "freeze_strategy")):
            return self.generate_diffusion_style(input_ids, generation_config, **kwargs)
        if any(k in kwargs for k in self._MINIMAL_LOOP_KEYS) or isinstance(generation_config, GenerationSettings):
            return self.generate_minimal(input_ids, generation_config, **kwargs)
        if generation_config is not None:
            kwargs["generation_config"] = generation_config
        return super().generate(input_ids, **kwargs)

    def generate_diffusion_style(self, input_ids: torch.Tensor, generation_config=None, **kwargs):
        """RMM:1234-1549; see diffusion.generate_diffusion_style."""
        from . import diffusion
        return diffusion.generate_diffusion_style(self, input_ids, generation_config, **kwargs)

    def generate_with_adaptive_compute(self, input_ids: torch.Tensor, generation_config=None, **kwargs):
        """RMM:1552-1749; see adaptive.generate_with_adaptive_compute."""
        from . import adaptive
        return adaptive.generate_with_adaptive_compute(self, input_ids, generation_config, **kwargs)

    def generate_speculative(self, input_ids: torch.Tensor, generation_config=None, **kwargs):
        """RMM:1750-1927; see speculative.generate_speculative."""
        from . import speculative
        return speculative.generate_speculative(self, input_ids, generation_config, **kwargs)

    def forward_with_adaptive_compute(self, input_ids: torch.Tensor, exit_evaluator, **kwargs):
        """RMM:998-1035; see adaptive.forward_with_adaptive_compute."""
        from . import adaptive
        return adaptive.forward_with_adaptive_compute(self, input_ids, exit_evaluator, **kwargs)

    def _prefill_with_varied_exit_steps(self, input_ids: torch.Tensor, exit_evaluator, past_key_values=None,
                                        init_scale: float = 1.0, **kwargs):
        """RMM:937-996; see adaptive.prefill_with_varied_exit_steps."""
        from . import adaptive
        return adaptive.prefill_with_varied_exit_steps(self, input_ids, exit_evaluator, past_key_values, init_scale, **kwargs)

    @torch.no_grad()
    def generate_minimal(self, input_ids: torch.Tensor, generation_config=None, tokenizer=None, streamer=None,
                         continuous_compute: bool = False, init_scale: float = 1.0, cache_lookup_strategy: str = "full",
                         input_states_fn: Optional[Callable] = None, stop_tokens: Optional[set] = None,
                         use_graph: bool = True, **model_kwargs):
        """RMM:1165-1232.  Prefill through forward(), then one token per step through the decode
        runner (all kernels of a token on one stream, optionally replayed as a HIP graph).

        input_states_fn(call_index, (B, S, h)) -> latent state to inject into that forward (an
        extension for reproducible runs: the reference re-draws the state from the device RNG on
        every call, RMM:738).  stop_tokens overrides the reference's fixed stop set."""
        gc = generation_config if generation_config is not None else self.generation_config
        B, prompt_len = input_ids.shape
        if "max_new_tokens" in model_kwargs and model_kwargs["max_new_tokens"] is not None:
            max_new = model_kwargs["max_new_tokens"]
            if "max_length" in model_kwargs:
                max_new = min(max_new, model_kwargs["max_length"] - prompt_len)
        elif getattr(gc, "max_new_tokens", None):
            max_new = gc.max_new_tokens
        else:
            max_new = model_kwargs.get("max_length", self._default_max_length(gc)) - prompt_len
        num_steps = model_kwargs.get("num_steps", None)
        stops = self._get_stops(gc) if stop_tokens is None else set(stop_tokens)
        input_ids = input_ids.to(self.device)
        if max_new <= 0:
            return input_ids
        total = min(prompt_len + max_new, self.config.block_size)
        cache = self._generation_cache(model_kwargs, cache_lookup_strategy, B, total)

        def state_for(call: int, S: int, embeds_like=None):
            if input_states_fn is not None:
                return input_states_fn(call, (B, S, self.config.n_embd)).to(self.device, self.dtype)
            return None

        # prefill
        seen = cache.get_seq_length()
        pos = torch.arange(seen, prompt_len, device=self.device)
        out = self.forward(input_ids=input_ids[:, seen:], input_states=state_for(0, prompt_len - seen), num_steps=num_steps,
                           past_key_values=cache, use_cache=True, cache_position=pos, init_scale=init_scale)
        next_tok = self._sample_next_token(out.logits[:, -1, :], input_ids, gc)
        carried = out.latent_states[:, -1:, :] if continuous_compute else None
        tokens = [next_tok]
        alive = torch.ones(B, dtype=torch.bool)
        if streamer:
            streamer.put(next_tok.cpu())

        def update_alive(tok) -> bool:
            if stops:
                for b, v in enumerate(tok.view(-1).tolist()):
                    if alive[b] and v in stops:
                        alive[b] = False
            return bool(alive.any())

        runner = None
        call = 1
        # the penalties look at the growing sequence on every step (RMM:1198-1201, 1946-1947); with one configured the
        # pick is made from the penalised logits on the greedy path too
        penalised = getattr(gc, "repetition_penalty", None) is not None and gc.repetition_penalty != 1.0
        pick_on_host = bool(getattr(gc, "do_sample", False)) or penalised
        all_ids = torch.cat([input_ids, next_tok], dim=-1) if pick_on_host else None
        while len(tokens) < max_new and update_alive(tokens[-1]) and cache.get_seq_length() + 1 <= total:
            if runner is None:
                runner = DecodeRunner(self, cache, B, self._split_steps(num_steps), greedy=not getattr(gc, "do_sample", False),
                                      use_graph=use_graph)
            state = carried if continuous_compute else state_for(call, 1)
            logits, nxt, latents = runner.step(tokens[-1].view(-1), state, init_scale)
            if pick_on_host:
                nxt = self._sample_next_token(logits, all_ids, gc).view(-1)
                all_ids = torch.cat([all_ids, nxt.view(B, 1)], dim=-1)
            tokens.append(nxt.view(B, 1).clone())
            if continuous_compute:
                carried = latents.view(B, 1, -1).clone()
            if streamer:
                streamer.put(tokens[-1].cpu())
            call += 1
        if streamer:
            streamer.end()
        sequences = torch.cat([input_ids] + tokens, dim=-1)
        if getattr(gc, "return_dict_in_generate", False):
            return GenerateOutput(sequences=sequences, past_key_values=cache, scores={})
        return sequences


class DecodeRunner:
    """One decode step (S = 1) with every buffer preallocated: embedding, prelude, r recurrences,
    coda, ln_f, LM head and greedy argmax are enqueued back to back on the current stream.  The
    position is read by the kernels from a device counter, so the identical launch sequence serves
    every token and can be replayed as one HIP graph."""

    def __init__(self, model: RavenForCausalLM, cache: HuginnDynamicCache, batch: int, num_steps: int, greedy: bool = True,
                 use_graph: bool = True):
        cfg = model.config
        self.model, self.cache, self.B, self.r, self.greedy = model, cache, batch, num_steps, greedy
        dev, dt, h = model.device, model.dtype, cfg.n_embd
        n_pos = cfg.n_layers_in_prelude + cfg.n_layers_in_recurrent_block * num_steps
        n_pos = max((remap_step(s, cache.lookup_strategy) for s in range(n_pos)), default=-1) + 1
        need_t = cache.max_length if cache.max_length is not None else cache.get_seq_length() + 1
        cache.ensure(max(n_pos, 1), cfg.n_layers_in_coda, batch, cfg.n_heads, cfg.head_dim, need_t, dt, dev)
        self.ids = torch.zeros(batch, dtype=torch.int64, device=dev)
        self.pos = torch.zeros(1, dtype=torch.int32, device=dev)
        self.state = torch.zeros(batch, h, dtype=dt, device=dev)
        self.embeds = torch.empty(batch, h, dtype=dt, device=dev)
        self.x = torch.empty(batch, h, dtype=dt, device=dev)
        self.y = torch.empty(batch, h, dtype=dt, device=dev)
        self.latents = torch.empty(batch, h, dtype=dt, device=dev)
        self.logits = torch.empty(batch, cfg.padded_vocab_size, dtype=torch.float32, device=dev)
        self.next_ids = torch.zeros(batch, dtype=torch.int64, device=dev)
        if batch >= 17 and model.dtype == torch.bfloat16 and model.pack_chunk_weights:
            model.pack_weights()  # decode steps of 17..32 rows read Wqkv and mlp.fc through their line-aligned copies
        self.ws = hip.block_workspace(model._natives()["dims"], batch, dev)
        self.use_graph = use_graph and cfg.test_time_noise <= 0  # the noise draws are not part of a replayable launch sequence
        self.graph: Optional[torch.cuda.CUDAGraph] = None
        self._graph_key = None
        self._warm = False

    def _slots(self):
        """(prelude slots, first core slot per recurrence or per-block slots, coda slots) for one token."""
        cfg, c = self.model.config, self.cache
        n_pre, n_core, n_coda = cfg.n_layers_in_prelude, cfg.n_layers_in_recurrent_block, cfg.n_layers_in_coda
        pre = [c._slot(remap_step(i, c.lookup_strategy)) for i in range(n_pre)]
        core = [[c._slot(remap_step(n_pre + it * n_core + j, c.lookup_strategy)) for j in range(n_core)] for it in range(self.r)]
        coda = [c._slot(-(i + 1)) for i in range(n_coda)]
        return pre, core, coda

    # positions (the new one included) up to which the library runs the decode attention of two rows and more as one
    # workgroup per (head, row) instead of splitting the positions over workgroups (its "attn_nosplit_len" default)
    SHORT_CACHE_POSITIONS = 1536

    def _position_bound(self, pos0: int) -> int:
        """The by-value position that sizes the grids of a step at position pos0; the kernels take the true position
        from the device.  It is the cache's capacity, except while the sequence is short enough for the unsplit decode
        attention: then it is that rule's limit, so that a cache sized for a long generation does not cost a short
        sequence the split launch and its merge (the step's graph is captured again once, when the sequence crosses)."""
        cap = self.cache.t_max - 1
        return cap if pos0 + 1 > self.SHORT_CACHE_POSITIONS else min(cap, self.SHORT_CACHE_POSITIONS - 1)

    def _enqueue(self, hint: int):
        """Launches one token's kernels; reads the position from self.pos.  hint bounds the position for grid sizing."""
        m, t = self.model, self.model.transformer
        nat, cfg, B = m._natives(), m.config, self.B
        kv = self.cache.native()
        pre, core, coda = self._slots()
        hip.embed(t.wte.weight, self.ids, m.emb_scale, out=self.embeds)
        cur = self.embeds
        for i, slot in enumerate(pre):
            hip.sandwich_block(nat["dims"], nat["prelude"][i], cur, self.embeds, nat["freqs"], kv, slot, B, 1, hint, self.ws,
                               pos_dev=self.pos)
        x = self.state
        n_core = len(t.core_block)
        if n_core > 0 and self.r > 0 and cfg.test_time_noise > 0:
            # the state is perturbed in front of every recurrence (RMM:775): one call per recurrence
            for it in range(self.r):
                x = m._maybe_inject_noise(x, it)
                hip.core_iterations(nat["dims"], t.adapter.weight, nat["core"], x, self.embeds, self.x, nat["freqs"], kv, [core[it]], B, 1,
                                    hint, self.ws, ln_f=t.ln_f.weight if it == self.r - 1 else None, pos_dev=self.pos)
                x = self.x
        elif n_core > 0 and self.r > 0:
            # all recurrences in one call: for one row the library folds each closing norm into the next adapter product
            hip.core_iterations(nat["dims"], t.adapter.weight, nat["core"], x, self.embeds, self.x, nat["freqs"], kv, core, B, 1, hint,
                                self.ws, ln_f=t.ln_f.weight, pos_dev=self.pos)
            x = self.x
        elif self.r > 0:
            raise NotImplementedError("the decode runner needs at least one core block; use forward() for such a model")
        if self.r == 0:
            hip.load().raven_rmsnorm_residual(x.data_ptr(), None, t.ln_f.weight.data_ptr(), self.x.data_ptr(), None, None, None,
                                              B, cfg.n_embd, cfg.norm_eps, hip.dtype_code(m.dtype), hip._stream())
            x = self.x
        self.latents.copy_(x)
        n_coda = len(coda)
        for i, slot in enumerate(coda):
            hip.sandwich_block(nat["dims"], nat["coda"][i], x, self.y, nat["freqs"], kv, slot, B, 1, hint, self.ws,
                               ln_f=t.ln_f.weight if i == n_coda - 1 else None, pos_dev=self.pos)
            x = self.y
        if n_coda == 0:
            hip.load().raven_rmsnorm_residual(x.data_ptr(), None, t.ln_f.weight.data_ptr(), self.y.data_ptr(), None, None, None,
                                              B, cfg.n_embd, cfg.norm_eps, hip.dtype_code(m.dtype), hip._stream())
            x = self.y
        rc = hip.load().raven_gemm(x.data_ptr(), m.lm_head.weight.data_ptr(), None, self.logits.data_ptr(), B,
                                   cfg.padded_vocab_size, cfg.n_embd, hip.dtype_code(m.dtype), 1, hip._stream())
        hip._check(rc, "raven_gemm")
        hip.argmax(self.logits, out=self.next_ids)
        hip.advance_pos(self.pos, 1)

    def step(self, ids: torch.Tensor, state: Optional[torch.Tensor], init_scale: float = 1.0):
        """Feeds one token per sequence; returns (logits [B,V] f32, next ids [B], latents [B,h]).
        The returned tensors are the runner's own buffers: copy what must outlive the next step."""
        m, c = self.model, self.cache
        pos0 = c._seen_tokens
        if pos0 + 1 > m.config.block_size:
            raise ValueError(f"position {pos0} lies past the RoPE table (block_size {m.config.block_size})")
        last_step = m.config.n_layers_in_prelude + m.config.n_layers_in_recurrent_block * self.r - 1
        if c.has_gap(last_step, pos0):
            raise NotImplementedError("the decode runner's fixed launch sequence needs a cache whose earlier tokens were all "
                                      f"computed with at least {self.r} recurrences; use forward() for partially filled caches")
        if pos0 + 1 > c.t_max or (c.max_length is not None and pos0 + 1 > c.max_length):
            c.ensure(1, 0, self.B, m.config.n_heads, m.config.head_dim, pos0 + 1, m.dtype, m.device)  # grows (pointers move), or refuses past max_length
            self.graph = None
        hint = self._position_bound(pos0)
        if self.B >= 17 and m.dtype == torch.bfloat16 and m.pack_chunk_weights:
            m.pack_weights()  # no work unless a weight changed since the copies were made (in place: the copies keep their addresses)
        self.ids.copy_(ids.view(-1))
        self.pos.fill_(pos0)
        if state is None:
            if init_scale > 0:
                self.state.copy_(m.initialize_state(self.embeds, init_scale))
            else:
                self.state.zero_()
        else:
            self.state.copy_(state.reshape(self.B, -1))
        if self.use_graph and self._warm:
            # the captured launches hold the cache's pointers, slot numbers and capacity: any reallocation (more
            # positions, more step slots) makes them stale
            key = (c._k.data_ptr(), c._v.data_ptr(), tuple(c._k.shape), c._neg_slots, hint)
            if self.graph is None or self._graph_key != key:
                self.graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(self.graph):
                    self._enqueue(hint)
                self._graph_key = key
                self.pos.fill_(pos0)  # capture does not execute; make sure the counter is what this step needs
            self.graph.replay()
        else:
            self._enqueue(hint)
            self._warm = True
        # bookkeeping the reference does inside cache.update (RMM:188-196)
        cfg = m.config
        c._seen_tokens += 1
        n_steps = cfg.n_layers_in_prelude + cfg.n_layers_in_recurrent_block * self.r
        for s in list(range(n_steps)) + [-(i + 1) for i in range(cfg.n_layers_in_coda)]:
            c.note_append(s, 1, pos0)
        return self.logits, self.next_ids, self.latents



# ---- transformers registration (RMM:2312-2323) -----------------------------------------------------
RavenConfig.register_for_auto_class()
RavenForCausalLM.register_for_auto_class("AutoModel")
RavenForCausalLM.register_for_auto_class("AutoModelForCausalLM")
AutoConfig.register("huginn_raven", RavenConfig, exist_ok=True)
AutoModel.register(RavenConfig, RavenForCausalLM, exist_ok=True)
AutoModelForCausalLM.register(RavenConfig, RavenForCausalLM, exist_ok=True)
