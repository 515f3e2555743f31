"""Decode over block-paged KV caches: what the model of the reference's vLLM plugin does for a batch of decode rows
(RavenModel.forward, vllm/raven_vllm.py:374-411), without vLLM.

Every flat layer (prelude, core and coda blocks in forward order) owns ONE paged cache [num_blocks, block_size, n_heads,
head_dim] for keys and one for values; the recurrences of a token overwrite the core layers' entries in turn, so older
positions hold the keys and values of their last recurrence -- the cache sharing that the Hugging Face surface calls
`latest-m4-compress-s4` (raven_modeling_minimal.py:169-182), which is why a prompt processed through that surface can be
copied into the pages (`load_prompt`).  A sequence is a row of the block table plus a length; sequences of different
lengths decode together, each at its own position (the contiguous cache of the Hugging Face surface shares one position
across the batch, raven_modeling_minimal.py:660-665).

The arithmetic of a step is the contiguous decode path's: the same SandwichBlock launches with the paged decode-attention
kernel in place of the contiguous one (raven_paged_decode_blocks).  forward_tokens takes any mix of prompt chunks and decode
rows of several sequences, flattened as a serving engine hands them over, through the paged chunk kernels
(raven_paged_qkv_rope_append, raven_paged_prefill_attention)."""

from __future__ import annotations

from typing import Optional, Sequence

import torch

from . import hip
from .cache import HuginnDynamicCache, remap_step

PAGED_STRATEGY = "latest-m4-compress-s4"


class PagedDecoder:
    def __init__(self, model, num_blocks: int, block_size: int = 16, num_steps: Optional[int] = None, use_graph: bool = False,
                 layout: str = "HND"):
        cfg = model.config
        self.model, self.cfg = model, cfg
        self.r = cfg.mean_recurrence if num_steps is None else int(num_steps)
        if self.r < 1:
            raise ValueError("num_steps must be at least 1")
        self.block_size, self.num_blocks = int(block_size), int(num_blocks)
        dev, dt = model.device, model.dtype
        self.n_flat = cfg.n_layers_in_prelude + cfg.n_layers_in_recurrent_block + cfg.n_layers_in_coda
        # "NHD": [num_blocks, block_size, n_heads, head_dim]; "HND": [num_blocks, n_heads, block_size, head_dim], where a
        # head's positions of a block are contiguous (the attention kernel reads it about 15 % faster)
        if layout not in ("NHD", "HND"):
            raise ValueError(f"unknown layout {layout!r}")
        self.layout = hip.PAGED_NHD if layout == "NHD" else hip.PAGED_HND
        shape = ((self.num_blocks, self.block_size, cfg.n_heads, cfg.head_dim) if layout == "NHD" else
                 (self.num_blocks, cfg.n_heads, self.block_size, cfg.head_dim))
        self.k = [torch.zeros(shape, dtype=dt, device=dev) for _ in range(self.n_flat)]
        self.v = [torch.zeros(shape, dtype=dt, device=dev) for _ in range(self.n_flat)]
        self._ws = {}
        # use_graph: a step's launches are captured once per (batch size, table width) and replayed; ids, block table,
        # lengths and latent state are copied into fixed buffers that the captured kernels read
        self.use_graph = use_graph

    # ------------------------------------------------------------------ prompts
    def _flat_steps(self):
        """Step index, in the other surface's cache, of each flat layer's final entries."""
        cfg = self.cfg
        n_pre, n_core = cfg.n_layers_in_prelude, cfg.n_layers_in_recurrent_block
        last = n_pre + (self.r - 1) * n_core
        return ([i for i in range(n_pre)] + [remap_step(last + j, PAGED_STRATEGY) for j in range(n_core)] +
                [-(i + 1) for i in range(cfg.n_layers_in_coda)])

    def load_prompt(self, cache: HuginnDynamicCache, row: int, table_row: Sequence[int]) -> int:
        """Copies sequence `row` of a cache filled through the other surface with lookup_strategy `latest-m4-compress-s4`
        into the pages listed in table_row; returns the number of positions."""
        if (self.cfg.n_layers_in_prelude, self.cfg.n_layers_in_recurrent_block) != (2, 4):
            # the equivalence with the cache-sharing strategy of the other surface hard-codes these counts (RMM:169-182)
            raise NotImplementedError("prompts come over from the other surface only for a model with 2 prelude and 4 core blocks; "
                                      "forward_tokens() has no such limit")
        if cache.lookup_strategy != PAGED_STRATEGY:
            raise ValueError(f"a prompt for the paged decoder must be cached with lookup_strategy={PAGED_STRATEGY!r}")
        n = cache.get_seq_length()
        if n > len(table_row) * self.block_size:
            raise ValueError(f"{len(table_row)} blocks of {self.block_size} cannot hold {n} positions")
        pos = torch.arange(n)
        table = torch.as_tensor(list(table_row), dtype=torch.int64)
        slots = (table[pos // self.block_size] * self.block_size + pos % self.block_size).to(self.model.device)
        h = self.cfg.n_heads * self.cfg.head_dim
        for f, step in enumerate(self._flat_steps()):
            s = cache._slot(step)
            k = cache._k[s, row, :, :n].transpose(0, 1).reshape(n, h).contiguous()
            v = cache._v[s, row, :, :n].transpose(0, 1).reshape(n, h).contiguous()
            hip.paged_kv_append(k, v, self.k[f], self.v[f], slots, layout=self.layout)
        return n

    def prefill(self, input_ids: torch.Tensor, table_row: Sequence[int], input_states: Optional[torch.Tensor] = None):
        """One prompt [1, n] through the chunk kernels of the other surface, then into the pages.  Returns its output."""
        cache = HuginnDynamicCache(lookup_strategy=PAGED_STRATEGY)
        n = input_ids.shape[1]
        out = self.model(input_ids=input_ids, input_states=input_states, past_key_values=cache, use_cache=True,
                         cache_position=torch.arange(n, device=input_ids.device), num_steps=self.r)
        self.load_prompt(cache, 0, table_row)
        return out

    # ------------------------------------------------------------------ rows of any sequences (prompt chunks, decode rows)

    def _token_block(self, blk, f: int, x: torch.Tensor, meta) -> torch.Tensor:
        """One SandwichBlock (vllm/raven_vllm.py:289-294 around its attention layer, :184-203) on flat rows, flat layer f."""
        eps = self.cfg.norm_eps
        positions, slots, table, lens, q_start, max_q = meta
        n1 = hip.rmsnorm_residual(x, blk.norm_1.weight, eps)[0]
        qkv = hip.linear(n1, blk.attn.Wqkv.weight)
        bias = blk.attn.qk_bias if hasattr(blk.attn, "qk_bias") else None
        q = hip.paged_qkv_rope_append(qkv, bias, self.model._natives()["freqs"], positions, slots, self.k[f], self.v[f], layout=self.layout)
        ya = hip.paged_prefill_attention(q, self.k[f], self.v[f], table, lens, q_start, max_q, layout=self.layout)
        # the residual adds (RMM:534-535) and the SwiGLU (RMM:507-508) ride in the epilogues of the products
        x1 = hip.linear(ya, blk.attn.proj.weight, residual=x)
        x2, _, n3 = hip.rmsnorm_residual(x1, blk.norm_2.weight, eps, weight2=blk.norm_3.weight)
        x3 = hip.linear(hip.linear(n3, blk.mlp.fc.weight, swiglu=True), blk.mlp.proj.weight, residual=x2)
        return hip.rmsnorm_residual(x3, blk.norm_4.weight, eps)[0]

    @torch.no_grad()
    def forward_tokens(self, input_ids: torch.Tensor, positions: torch.Tensor, slot_mapping: torch.Tensor, block_table: torch.Tensor,
                       seq_lens: torch.Tensor, query_start_loc: torch.Tensor, max_query_len: int,
                       input_states: Optional[torch.Tensor] = None, init_scale: float = 1.0, check_bounds: Optional[bool] = None):
        """What the plugin's model computes for one scheduler step (RavenModel.forward, vllm/raven_vllm.py:374-411), straight on
        the pages: input_ids [T] are the new rows of B sequences, flattened (prompt chunks of any length and decode rows
        together); positions [T] and slot_mapping [T] (int64) say where each row sits; sequence b owns rows
        query_start_loc[b] .. query_start_loc[b + 1] - 1 and holds seq_lens[b] positions once they are appended.
        Returns (logits [T, V] float32, latents [T, h]).  bf16 models with head_dim 64 / 96 / 128."""
        m, cfg, t = self.model, self.cfg, self.model.transformer
        if m.dtype != torch.bfloat16:
            raise NotImplementedError("forward_tokens: the paged chunk attention kernel is bf16 only")
        T = input_ids.numel()
        B = seq_lens.shape[0]
        if positions.shape != (T,) or slot_mapping.shape != (T,) or query_start_loc.shape != (B + 1,) or block_table.shape[0] != B:
            raise ValueError("positions [T], slot_mapping [T], block_table [B, max_blocks], seq_lens [B], query_start_loc [B + 1]")
        if self._wants_check(check_bounds, block_table, seq_lens, positions, slot_mapping):
            self._check_pages(block_table, seq_lens, positions, slot_mapping)
        dev = m.device
        meta = (positions.to(dev, torch.int64), slot_mapping.to(dev, torch.int64), block_table.to(dev, torch.int32).contiguous(),
                seq_lens.to(dev, torch.int32), query_start_loc.to(dev, torch.int32), int(max_query_len))
        n_pre, n_core = cfg.n_layers_in_prelude, cfg.n_layers_in_recurrent_block
        x = hip.embed(t.wte.weight, input_ids.reshape(-1).to(dev, torch.int64).contiguous(), m.emb_scale)
        for i in range(n_pre):
            x = self._token_block(t.prelude[i], i, x, meta)
        embeds = x
        if input_states is None:
            state = m.initialize_state(embeds, init_scale) if init_scale > 0 else torch.zeros_like(embeds)
        else:
            state = input_states.reshape(T, -1).to(dev, m.dtype)
        for _ in range(self.r):
            state = hip.linear(state, t.adapter.weight, x1=embeds)  # the concat of RMM:776 as two K segments
            for j in range(n_core):
                state = self._token_block(t.core_block[j], n_pre + j, state, meta)
        latents = hip.rmsnorm_residual(state, t.ln_f.weight, cfg.norm_eps)[0]
        x = latents
        for i in range(cfg.n_layers_in_coda):
            x = self._token_block(t.coda[i], n_pre + n_core + i, x, meta)
        x = hip.rmsnorm_residual(x, t.ln_f.weight, cfg.norm_eps)[0]
        logits = hip.gemm(x, m.lm_head.weight, out_f32=True)
        return logits, latents

    def prefill_paged(self, input_ids: torch.Tensor, table_row: Sequence[int], input_states: Optional[torch.Tensor] = None,
                      chunk: Optional[int] = None):
        """One prompt [1, n] straight into the pages of table_row, `chunk` rows at a time (all at once by default).
        Returns (logits [n, V], latents [n, h])."""
        n = input_ids.shape[1]
        if n > len(table_row) * self.block_size:
            raise ValueError(f"{len(table_row)} blocks of {self.block_size} cannot hold {n} positions")
        chunk = n if chunk is None else int(chunk)
        table = torch.as_tensor([list(table_row)], dtype=torch.int32)
        row = torch.as_tensor(list(table_row), dtype=torch.int64)
        outs = []
        for lo in range(0, n, chunk):
            hi = min(n, lo + chunk)
            pos = torch.arange(lo, hi)
            slots = row[pos // self.block_size] * self.block_size + pos % self.block_size
            st = None if input_states is None else input_states[:, lo:hi]
            outs.append(self.forward_tokens(input_ids[0, lo:hi], pos, slots, table, torch.tensor([hi], dtype=torch.int32),
                                            torch.tensor([0, hi - lo], dtype=torch.int32), hi - lo, input_states=st))
        return torch.cat([o[0] for o in outs]), torch.cat([o[1] for o in outs])

    # ------------------------------------------------------------------ decode
    def _buffers(self, B: int, max_blocks: int):
        key = (B, max_blocks)
        if key not in self._ws:
            m, cfg = self.model, self.cfg
            dev, dt, h = m.device, m.dtype, cfg.n_embd
            nat = m._natives()
            if B >= 17 and dt == torch.bfloat16 and m.pack_chunk_weights:
                m.pack_weights()  # decode steps of 17..32 rows read Wqkv and mlp.fc through their line-aligned copies
            mk = lambda: torch.empty(B, h, dtype=dt, device=dev)
            self._ws[key] = {
                "ids": torch.zeros(B, dtype=torch.int64, device=dev),
                "table": torch.zeros(B, max_blocks, dtype=torch.int32, device=dev),
                "lens": torch.zeros(B, dtype=torch.int32, device=dev),
                "state": mk(), "embeds": mk(), "pre": mk(), "x": mk(), "y": mk(),
                "logits": torch.empty(B, cfg.padded_vocab_size, dtype=torch.float32, device=dev),
                "ws": hip.block_workspace(nat["dims"], B, dev),
                "graph": None, "warm": False,
            }
        return self._ws[key]

    def _enqueue(self, buf, B: int):
        m, cfg, t = self.model, self.cfg, self.model.transformer
        nat = m._natives()
        max_len = buf["table"].shape[1] * self.block_size  # sizes the launch only; lengths are read on the device
        n_pre, n_core = cfg.n_layers_in_prelude, cfg.n_layers_in_recurrent_block
        kvs = [hip.make_paged_kv(self.k[a:b], self.v[a:b], buf["table"], buf["lens"], max_len, layout=self.layout)
               for a, b in ((0, n_pre), (n_pre, n_pre + n_core), (n_pre + n_core, self.n_flat))]
        hip.embed(t.wte.weight, buf["ids"], m.emb_scale, out=buf["embeds"])
        pre = (hip.BlockWeights * n_pre)(*nat["prelude"])
        hip.paged_decode_blocks(nat["dims"], pre, buf["embeds"], buf["pre"], nat["freqs"], kvs[0], B, buf["ws"])
        hip.paged_decode_blocks(nat["dims"], nat["core"], buf["state"], buf["x"], nat["freqs"], kvs[1], B, buf["ws"],
                                adapter_w=t.adapter.weight, embeds=buf["pre"], n_iterations=self.r, ln_f=t.ln_f.weight)
        if cfg.n_layers_in_coda > 0:
            coda = (hip.BlockWeights * cfg.n_layers_in_coda)(*nat["coda"])
            hip.paged_decode_blocks(nat["dims"], coda, buf["x"], buf["y"], nat["freqs"], kvs[2], B, buf["ws"], ln_f=t.ln_f.weight)
        else:
            rc = hip.load().raven_rmsnorm_residual(buf["x"].data_ptr(), None, t.ln_f.weight.data_ptr(), buf["y"].data_ptr(), None, None,
                                                   None, B, cfg.n_embd, cfg.norm_eps, hip.dtype_code(m.dtype), hip._stream())
            hip._check(rc, "raven_rmsnorm_residual")
        rc = hip.load().raven_gemm(buf["y"].data_ptr(), m.lm_head.weight.data_ptr(), None, buf["logits"].data_ptr(), B,
                                   cfg.padded_vocab_size, cfg.n_embd, hip.dtype_code(m.dtype), 1, hip._stream())
        hip._check(rc, "raven_gemm")

    @staticmethod
    def _wants_check(check_bounds: Optional[bool], *tensors) -> bool:
        if check_bounds is not None:
            return check_bounds
        return all(t is None or t.device.type == "cpu" for t in tensors)

    def _check_pages(self, block_table: torch.Tensor, seq_lens: torch.Tensor, positions: Optional[torch.Tensor] = None,
                     slot_mapping: Optional[torch.Tensor] = None) -> None:
        """The kernels index the RoPE table by position and the pages through the block table without looking: whatever
        they will dereference is checked here, on host copies (one device-to-host read when the tensors live on the GPU)."""
        lens = seq_lens.detach().to("cpu", torch.int64)
        table = block_table.detach().to("cpu", torch.int64)
        n_pos = self.cfg.block_size  # rows of the RoPE table
        if lens.numel() and (int(lens.min()) < 0 or int(lens.max()) > n_pos):
            raise ValueError(f"seq_lens must lie in [0, {n_pos}] (the RoPE table has {n_pos} positions); got up to {int(lens.max())}")
        if lens.numel() and int(lens.max()) > table.shape[1] * self.block_size:
            raise ValueError(f"a sequence of {int(lens.max())} positions does not fit {table.shape[1]} blocks of {self.block_size}")
        used = (lens + self.block_size - 1) // self.block_size
        mask = torch.arange(table.shape[1])[None, :] < used[:, None]
        if mask.any():
            ids = table[mask]
            if int(ids.min()) < 0 or int(ids.max()) >= self.num_blocks:
                raise ValueError(f"block_table names block {int(ids.max() if ids.max() >= self.num_blocks else ids.min())}; "
                                 f"the caches have {self.num_blocks}")
        if positions is not None and positions.numel():
            pos = positions.detach().to("cpu", torch.int64)
            if int(pos.min()) < 0 or int(pos.max()) >= n_pos:
                raise ValueError(f"positions must lie in [0, {n_pos}); got {int(pos.min())} .. {int(pos.max())}")
        if slot_mapping is not None and slot_mapping.numel():
            slots = slot_mapping.detach().to("cpu", torch.int64)
            if int(slots.max()) >= self.num_blocks * self.block_size:
                raise ValueError(f"slot_mapping names slot {int(slots.max())}; the caches have {self.num_blocks * self.block_size}")

    def step(self, ids: torch.Tensor, block_table: torch.Tensor, seq_lens: torch.Tensor, input_states: Optional[torch.Tensor] = None,
             init_scale: float = 1.0, check_bounds: Optional[bool] = None):
        """One new token per sequence.  ids [B]; block_table [B, max_blocks] int32; seq_lens [B] int32 = each sequence's
        length INCLUDING the new token (its position is seq_lens - 1; the page for it must be in the table).
        Returns (logits [B, V] float32, latents [B, h]); both are buffers reused by the next step of the same batch size.
        check_bounds: None (default) validates seq_lens / block_table when they arrive as CPU tensors, where looking costs
        nothing, and trusts tensors that already live on the GPU (validating those is a device-to-host read and a
        synchronisation per scheduler step); True validates either way, False never."""
        m = self.model
        B = ids.shape[0]
        if block_table.dim() != 2 or block_table.shape[0] != B or seq_lens.shape != (B,):
            raise ValueError("block_table [B, max_blocks] and seq_lens [B] must match ids [B]")
        if self._wants_check(check_bounds, block_table, seq_lens):
            self._check_pages(block_table, seq_lens)
        buf = self._buffers(B, block_table.shape[1])
        buf["ids"].copy_(ids.view(-1))
        buf["table"].copy_(block_table)
        buf["lens"].copy_(seq_lens)
        if input_states is None:
            if init_scale > 0:
                buf["state"].copy_(m.initialize_state(buf["state"], init_scale))
            else:
                buf["state"].zero_()
        else:
            buf["state"].copy_(input_states.reshape(B, -1))
        if self.use_graph and buf["warm"]:
            if buf["graph"] is None:
                buf["graph"] = torch.cuda.CUDAGraph()
                with torch.cuda.graph(buf["graph"]):
                    self._enqueue(buf, B)
            buf["graph"].replay()
        else:
            self._enqueue(buf, B)
            buf["warm"] = True
        return buf["logits"], buf["x"]
