"""Vivepel decoder over the engine ops (`ops/mixers.py`).

Per layer (W = width, residual stream x in fp32, activations in the engine dtype: bf16 or fp32):
  h  = gnorm(x; norm1)                               fused into the previous sublayer's closing kernel
  qk = h @ [Wq; Wk]^T + [bq; bk]                     one GEMM for queries and keys (vendor GEMM, bias epilogue)
  q, cache <- per-head RMS norm, rotary on the first rot_dims entries, append (keys normed + rotated;
             values = the keys as projected)         ops.mixers.headnorm_rope_append
  a  = attention(q, cache): chunked causal mask, soft-capped scores, softmax with a sink, the heads'
       weights mixed by `talk` before they meet the values          ops.mixers.chunk_attention
  x += ls1 * gnorm(a @ Wo^T; norm1b);  h = gnorm(x; norm2)           ops.mixers.post_norm_residual
  x += ls2 * gnorm(PolyNorm(h @ Wup^T) @ Wdown^T; norm2b)            ops.mixers.polynorm, post_norm_residual
then gnorm(x; final norm) on the sampled rows and the LM head.

Every layer has its own head counts, sizes, chunk and rotary constants (`config.LayerSpec`), so the
paged cache is one (k, v) pair of tensors per layer, [NB, G, BS, D] each, under one block table:
the block manager and the scheduler see a single pool of pages.  Prefill, chunked prefill, mixed
and decode steps all run this same forward; a decode step is shape-static, so the runner captures it
into hipGraphs per batch bucket like Llama's.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch
import torch.nn.functional as F

from .. import ops
from ..ops import mixers
from .config import VivepelConfig
from .llama import AttnMeta


class VivepelModel:
    supports_block_copy = False     # no sub-block KV copies (ops.kv_block_copy assumes Llama's cache layout)

    def __init__(self, cfg: VivepelConfig, weights: Dict[str, torch.Tensor], comm=None, tp_rank: int = 0,
                 tp_size: int = 1, ep_rank: int = 0, ep_size: int = 1):
        if tp_size != 1 or ep_size != 1:
            raise ValueError("Vivepel runs at TP = 1")
        self.cfg = cfg
        self.W = weights
        self.comm = comm
        self.tp_rank, self.tp_size = 0, 1
        self.device = weights["embed"].device
        self.dtype = weights["embed"].dtype
        self.vocab_offset = 0
        self.layers: List[dict] = []
        for i in range(cfg.num_layers):
            p = f"layers.{i}."
            self.layers.append({k[len(p):]: v for k, v in weights.items() if k.startswith(p)})
        # the runner's hooks shared with LlamaModel
        self.persistent = False
        self.mark_layer = -1
        self.mark_event = None
        self.fuse_decode_rope = False
        # debugging / tests: called with (layer index, residual stream [T, W] fp32) after every layer
        self.layer_hook = None

    # ---- the runner's model interface ----------------------------------------------------------
    def alloc_cache(self, num_blocks: int, block_size: int):
        """(k_cache, v_cache): one tensor per layer, [NB, G, BS, D], zero-filled (a masked lane may read
        any slot of a live page, so stale slots must be finite)."""
        ks, vs = [], []
        for L in self.cfg.layers:
            m = L.mixer
            ks.append(torch.zeros((num_blocks, m.kv_heads, block_size, m.dim), dtype=self.dtype, device=self.device))
            vs.append(torch.zeros((num_blocks, m.kv_heads, block_size, m.vdim), dtype=self.dtype, device=self.device))
        return ks, vs

    def persistent_ok(self, B: int = 1) -> bool:
        return False

    def persistent_err_word(self):
        return None

    def persistent_err(self) -> int:
        return 0

    # ---- forward -------------------------------------------------------------------------------
    def hidden_states(self, input_ids: torch.Tensor, meta: AttnMeta, k_cache, v_cache) -> torch.Tensor:
        """The residual stream after the last layer for every row: [T, W] fp32."""
        cfg = self.cfg
        eps, groups = cfg.norm_eps, cfg.norm_groups
        x = mixers.embed_f32(input_ids, self.W["embed"])
        q_starts = None if meta.is_decode else meta.q_starts
        last = len(self.layers) - 1
        h = mixers.group_rmsnorm(x, self.layers[0]["norm1"], groups, eps, out_dtype=self.dtype) if self.layers else None
        for li, (L, spec) in enumerate(zip(self.layers, cfg.layers)):
            if li == self.mark_layer and x.is_cuda:   # progress marker (engine lookahead timing)
                self.mark_event = torch.cuda.Event()
                self.mark_event.record()
            m = spec.mixer
            qk = F.linear(h, L["wqk"], L["bqk"])
            q = mixers.headnorm_rope_append(qk, L["q_norm"], L["k_norm"], L["inv_freq"], meta.positions,
                                            meta.slot_mapping, k_cache[li], v_cache[li], m.heads, m.kv_heads, m.dim,
                                            m.rot_dims, eps)
            a = mixers.chunk_attention(q, k_cache[li], v_cache[li], meta.block_tables, q_starts, meta.positions,
                                       meta.slot_mapping, L["talk"], m.chunk, m.scale, m.softcap, sink=True,
                                       max_q=0 if meta.is_decode else meta.max_q_len,
                                       num_decode=0 if meta.is_decode else meta.num_decode)
            y = F.linear(a, L["wo"])
            nxt = self.layers[li + 1]["norm1"] if li < last else None
            if spec.ff:
                h = mixers.post_norm_residual(x, y, L["norm1b"], L["ls1"], L["norm2"], groups, eps)
                z = mixers.polynorm(F.linear(h, L["w_up"]), L["act"], eps)
                h = mixers.post_norm_residual(x, F.linear(z, L["w_down"]), L["norm2b"], L["ls2"], nxt, groups, eps)
            else:
                h = mixers.post_norm_residual(x, y, L["norm1b"], L["ls1"], nxt, groups, eps)
            if self.layer_hook is not None:
                self.layer_hook(li, x)
        return x

    def forward(self, input_ids: torch.Tensor, meta: AttnMeta, k_cache, v_cache) -> torch.Tensor:
        """The final-normed hidden state of the rows `meta.logits_indices`: [S, W] in the engine dtype."""
        x = self.hidden_states(input_ids, meta, k_cache, v_cache)
        if not (meta.is_decode and meta.logits_indices.shape[0] == x.shape[0]):
            x = x.index_select(0, meta.logits_indices)
        return mixers.group_rmsnorm(x, self.W["norm"], self.cfg.norm_groups, self.cfg.norm_eps, out_dtype=self.dtype)

    def logits(self, hidden_last: torch.Tensor) -> torch.Tensor:
        return F.linear(hidden_last, self.W["lm_head"])

    def sample(self, hidden_last: torch.Tensor, mask_bits: Optional[torch.Tensor],
               mask_idx: Optional[torch.Tensor]) -> torch.Tensor:
        """Greedy next tokens under the SAFE_DECODE mask: [S] int32."""
        logits = self.logits(hidden_last)
        if logits.dtype == torch.bfloat16 and logits.shape[1] % 8 == 0:
            return ops.masked_argmax(logits, mask_bits, mask_idx)[0]
        # fp32 engine (the verification dtype): the same rule on the fp32 logits
        return ops.ref.masked_argmax(logits, mask_bits, mask_idx)[0]
