"""What a binding of these kernels into the reference's vLLM plugin (vllm/raven_vllm.py) needs on the host side and can
be built without vLLM itself: the mapping between the Hugging Face state-dict names and the plugin's flat layer names
(RavenForvLLM.load_weights, raven_vllm.py:471-542), and the order in which a forward walks the flat layers
(RavenModel.forward, raven_vllm.py:374-411).  The device side is raven_paged_kv_append / raven_paged_decode_attention
(hip.paged_kv_append, hip.paged_decode_attention) for the block-paged KV cache that vLLM's attention layer owns.

vLLM is not installed where this package is built and tested: nothing here imports it, and the plugin class itself
(a torch.nn.Module built from vLLM's parallel linear layers) is not part of the package."""

from __future__ import annotations

from typing import Dict, List, Tuple

import torch

from .config import RavenConfig

_LEAF = (("attn.Wqkv.weight", "self_attn.qkv_proj.weight"), ("attn.proj.weight", "self_attn.o_proj.weight"),
         ("attn.qk_bias", "self_attn.qk_bias"), ("mlp.fc.weight", "mlp.gate_up_proj.weight"),
         ("mlp.proj.weight", "mlp.down_proj.weight"))


def vllm_name(name: str, cfg: RavenConfig):
    """The plugin's parameter name for a Hugging Face state-dict name, or None for entries the plugin recomputes
    (raven_vllm.py:481-526).  Prelude, core and coda blocks become one flat list `model.layers.N`."""
    if "freqs_cis" in name:
        return None
    if name == "lm_head.weight":
        return "model.embed_tokens.weight" if cfg.tie_embeddings else "lm_head.weight"
    if name == "transformer.wte.weight":
        return "model.embed_tokens.weight"
    for group, first in (("prelude", 0), ("core_block", cfg.n_layers_in_prelude),
                         ("coda", cfg.n_layers_in_prelude + cfg.n_layers_in_recurrent_block)):
        prefix = f"transformer.{group}."
        if name.startswith(prefix):
            idx, rest = name[len(prefix):].split(".", 1)
            name = f"model.layers.{first + int(idx)}.{rest}"
            break
    else:
        name = name.replace("transformer.ln_f", "model.ln_f").replace("transformer.adapter", "model.adapter")
    for hf, vl in _LEAF:
        if name.endswith(hf):
            return name[:-len(hf)] + vl
    return name


def to_vllm_state_dict(state_dict: Dict[str, torch.Tensor], cfg: RavenConfig) -> Dict[str, torch.Tensor]:
    """Renames a Hugging Face state dict for the plugin; qk_bias [2, 1, nh, hd] loses its singleton axis
    (raven_vllm.py:173, 531-532).  Tied embeddings collapse onto model.embed_tokens.weight."""
    out: Dict[str, torch.Tensor] = {}
    for name, t in state_dict.items():
        new = vllm_name(name, cfg)
        if new is None:
            continue
        out[new] = t.squeeze(1) if new.endswith("self_attn.qk_bias") and t.dim() == 4 else t
    return out


def hf_name(name: str, cfg: RavenConfig) -> str:
    """Inverse of vllm_name for the plugin's parameter names."""
    if name == "model.embed_tokens.weight":
        return "transformer.wte.weight"
    for hf, vl in _LEAF:
        if name.endswith(vl):
            name = name[:-len(vl)] + hf
            break
    if name.startswith("model.layers."):
        idx, rest = name[len("model.layers."):].split(".", 1)
        i, n_pre, n_core = int(idx), cfg.n_layers_in_prelude, cfg.n_layers_in_recurrent_block
        if i < n_pre:
            return f"transformer.prelude.{i}.{rest}"
        if i < n_pre + n_core:
            return f"transformer.core_block.{i - n_pre}.{rest}"
        return f"transformer.coda.{i - n_pre - n_core}.{rest}"
    return name.replace("model.ln_f", "transformer.ln_f").replace("model.adapter", "transformer.adapter")


def flat_layer_schedule(cfg: RavenConfig, num_steps: int = None) -> List[Tuple[str, int]]:
    """The order in which one forward of the plugin walks its flat layers: ("layer", i) for a decoder layer,
    ("adapter", r) before the core layers of recurrence r, ("ln_f", 0 / 1) (raven_vllm.py:389-411).  Every flat layer
    owns ONE paged cache, shared by all recurrences -- the Hugging Face cache with `compress-s4` behaves the same."""
    r = cfg.mean_recurrence if num_steps is None else num_steps
    n_pre, n_core, n_coda = cfg.n_layers_in_prelude, cfg.n_layers_in_recurrent_block, cfg.n_layers_in_coda
    plan: List[Tuple[str, int]] = [("layer", i) for i in range(n_pre)]
    for it in range(r):
        plan.append(("adapter", it))
        plan += [("layer", n_pre + j) for j in range(n_core)]
    plan.append(("ln_f", 0))
    plan += [("layer", n_pre + n_core + j) for j in range(n_coda)]
    plan.append(("ln_f", 1))
    return plan
