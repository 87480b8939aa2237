"""Kafilorn decoder over the engine ops (`ops/mixers.py`).

The residual is S fp32 copies ("streams") of the row, x [T, S, W].  A sublayer q of a layer reads one mixed row
and updates every copy (hyper-connections; S = 1 with unit weights is the plain pre-norm residual):
  h = LayerNorm(sum_s in_q[s] x_s)                            ops.mixers.stream_norm / fused into the update before it
  x_r <- sum_s mix_q[s, r] x_s + out_q[r] * sublayer(h)       ops.mixers.stream_update (+ the next sublayer's h)

Mixers (activations in the engine dtype, bf16 or fp32; what is marked fp32 is fp32 in both):
  mLSTM            [q | k | v | g] = h @ w_proj^T (one vendor GEMM); log gates from h in fp32 (mlstm_gates);
                   the recurrence over the step's rows from / into the sequence's state slot, fp32 (mlstm_scan:
                   numerators and denominators); division, per-head RMS division, weight, sigmoid(g) gate
                   (headnorm_gate); output GEMM.
  latent attention [c_q | c | k_r] = h @ w_dn^T (one GEMM); RMS norm of c_q, RMS norm of c and rotary on k_r
                   appended to the paged cache (latent_prep); q = c_q @ w_uq^T; rotary on q's rotated part
                   and the unrotated parts carried into the latent space by a batched GEMM with w_uk
                   (rope_split_q, bmm); multi-query attention over the cached rows with a sliding window and a
                   per-head sink, the latent as the value (window_attention); w_uv by a batched GEMM; output GEMM.
                   A layer with kv_from reads that layer's cache and appends nothing.
Feed-forwards: dense down(relu(up h)^2); or experts chosen per token by a grouped router (moe_route), their
weighted sum in fp32 (moe_experts) plus a shared gated expert.

Cache: one paged tensor [NB, BS, kv_rank + rot_dim] per latent-attention layer that owns its latent (borrowing
layers alias it), under the engine's single block table.  State: per mLSTM layer (S [slots, H, Dv, D],
n [slots, H, D], m [slots, H]) fp32, indexed by the sequence's state slot (`AttnMeta.state_slots`); a row at
position 0 starts from zeros, so slots are reused without clearing.  Prefill, chunked prefill, mixed and decode
steps all run this forward; the decode step is shape-static and capturable.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch
import torch.nn.functional as F

from .. import ops
from ..ops import mixers
from .config import KafilornConfig
from .llama import AttnMeta


class KafilornModel:
    supports_block_copy = False     # no sub-block KV copies (ops.kv_block_copy assumes Llama's cache layout)
    supports_prefix_cache = False   # a recurrent state cannot be rebuilt from cached pages

    def __init__(self, cfg: KafilornConfig, weights: Dict[str, torch.Tensor], comm=None, tp_rank: int = 0,
                 tp_size: int = 1, ep_rank: int = 0, ep_size: int = 1):
        if tp_size != 1 or ep_size != 1:
            raise ValueError("Kafilorn runs at TP = 1")
        self.cfg = cfg
        self.W = weights
        self.comm = comm
        self.tp_rank, self.tp_size = 0, 1
        self.device = weights["embed"].device
        self.dtype = weights["embed"].dtype
        self.vocab_offset = 0
        self.streams = max(cfg.streams, 1)
        self.layers: List[dict] = []
        for i in range(cfg.num_layers):
            p = f"layers.{i}."
            self.layers.append({k[len(p):]: v for k, v in weights.items() if k.startswith(p)})
        self.state: List[Optional[tuple]] = [None] * cfg.num_layers
        # the runner's hooks shared with LlamaModel
        self.persistent = False
        self.mark_layer = -1
        self.mark_event = None
        self.fuse_decode_rope = False
        # debugging / tests: called with (layer index, the streams' sum [T, W] fp32) after every layer
        self.layer_hook = None

    # ---- the runner's model interface ----------------------------------------------------------
    def alloc_cache(self, num_blocks: int, block_size: int):
        """(k_cache, v_cache): per layer the latent cache [NB, BS, kv_rank + rot_dim] (None for an mLSTM layer, the
        owner's tensor for a borrowing layer), zero-filled; there is no separate value cache."""
        ks: List[Optional[torch.Tensor]] = []
        for L in self.cfg.layers:
            m = L.mixer
            if m.kind != "latent_attention":
                ks.append(None)
            elif m.kv_from >= 0:
                ks.append(ks[m.kv_from])
            else:
                ks.append(torch.zeros((num_blocks, block_size, m.kv_rank + m.rot_dim), dtype=self.dtype, device=self.device))
        return ks, [None] * len(ks)

    def alloc_state(self, num_slots: int) -> None:
        """Recurrent state for `num_slots` live sequences (fp32 in every engine dtype)."""
        for i, L in enumerate(self.cfg.layers):
            m = L.mixer
            if m.kind == "mlstm":
                z = dict(dtype=torch.float32, device=self.device)
                self.state[i] = (torch.zeros((num_slots, m.heads, m.vdim, m.dim), **z),
                                 torch.zeros((num_slots, m.heads, m.dim), **z), torch.zeros((num_slots, m.heads), **z))

    def persistent_ok(self, B: int = 1) -> bool:
        return False

    def persistent_err_word(self):
        return None

    def persistent_err(self) -> int:
        return 0

    # ---- sublayers -----------------------------------------------------------------------------
    def _mlstm(self, h, L, m, li, meta: AttnMeta):
        if self.state[li] is None or meta.state_slots is None:
            raise RuntimeError("mLSTM layer without state slots: the runner must call alloc_state and pass state_slots")
        HD, HV = m.heads * m.dim, m.heads * m.vdim
        proj = F.linear(h, L["w_proj"])                                # [T, q | k | v | g]
        gates = mixers.mlstm_gates(h, L["w_if"], L["b_if"], m.gate_cap, L.get("w_if_lp"))
        S, n, mx = self.state[li]
        o, den = mixers.mlstm_scan(proj, 0, HD, 2 * HD, gates, S, n, mx, meta.state_slots,
                                   None if meta.is_decode else meta.q_starts, meta.positions, m.heads, m.dim, m.vdim,
                                   m.dim ** -0.5)
        return F.linear(mixers.headnorm_gate(o, proj, 2 * HD + HV, L["hnorm"], m.heads, m.vdim, self.cfg.norm_eps,
                                             self.dtype, den), L["wo"])

    def _latent_attention(self, h, L, m, cache, meta: AttnMeta):
        T = h.shape[0]
        own = m.kv_from < 0
        proj = F.linear(h, L["w_dn"])
        cq = mixers.latent_prep(proj, m.q_rank, m.kv_rank, m.rot_dim, L["q_norm"], L.get("kv_norm"), L["inv_freq"],
                                meta.positions, meta.slot_mapping, cache if own else None, m.rot_dims, self.cfg.norm_eps)
        qn, qr = mixers.rope_split_q(F.linear(cq, L["w_uq"]), L["inv_freq"], meta.positions, m.heads, m.dim, m.rot_dim,
                                     m.rot_dims)
        q_lat = torch.bmm(qn, L["w_uk"])                               # [H, T, R]
        o_lat = mixers.window_attention(q_lat, qr, cache, meta.block_tables, None if meta.is_decode else meta.q_starts,
                                        meta.positions, meta.slot_mapping, L["sink"], m.window, m.scale)
        o = torch.bmm(o_lat, L["w_uv"].transpose(1, 2))                # [H, T, Dv]
        return F.linear(o.transpose(0, 1).reshape(T, m.heads * m.vdim), L["wo"])

    def _feed_forward(self, h, L, f):
        if f.kind == "dense":
            return F.linear(mixers.relu_sq(F.linear(h, L["w_up"])), L["w_down"])
        ids, w = mixers.moe_route(h, L["w_router"], L["correction"], f.top, f.groups, f.keep_groups)
        y = mixers.moe_experts(h, L["w_gu"], L["w_dn_e"], ids, w)      # fp32
        if f.shared_ff:
            y += F.linear(mixers.silu_mul(F.linear(h, L["ws_gu"])), L["ws_down"])
        return y

    # ---- forward -------------------------------------------------------------------------------
    def hidden_states(self, input_ids: torch.Tensor, meta: AttnMeta, k_cache, v_cache) -> torch.Tensor:
        """The residual streams after the last layer for every row: [T, S, W] fp32."""
        cfg, eps = self.cfg, self.cfg.norm_eps
        x = mixers.embed_streams(input_ids, self.W["embed"], cfg.embed_scale, self.streams)
        last = len(self.layers) - 1
        h = mixers.stream_norm(x, self.layers[0]["hc1_in"], self.layers[0]["norm1"], eps, self.dtype) if self.layers else None
        for li, (L, spec) in enumerate(zip(self.layers, cfg.layers)):
            if li == self.mark_layer and x.is_cuda:   # progress marker (engine lookahead timing)
                self.mark_event = torch.cuda.Event()
                self.mark_event.record()
            m, f = spec.mixer, spec.mlp
            y = self._mlstm(h, L, m, li, meta) if m.kind == "mlstm" else self._latent_attention(h, L, m, k_cache[li], meta)
            nxt = self.layers[li + 1] if li < last else None
            n_in, n_w = (nxt["hc1_in"], nxt["norm1"]) if nxt is not None else (None, None)
            if f is not None:
                h = mixers.stream_update(x, y, L["hc1_mix"], L["hc1_out"], L["hc2_in"], L["norm2"], eps, self.dtype)
                h = mixers.stream_update(x, self._feed_forward(h, L, f), L["hc2_mix"], L["hc2_out"], n_in, n_w, eps, self.dtype)
            else:
                h = mixers.stream_update(x, y, L["hc1_mix"], L["hc1_out"], n_in, n_w, eps, self.dtype)
            if self.layer_hook is not None:
                self.layer_hook(li, x.sum(1))
        return x

    def forward(self, input_ids: torch.Tensor, meta: AttnMeta, k_cache, v_cache) -> torch.Tensor:
        """The final-normed hidden state of the rows `meta.logits_indices`: [S, W] in the engine dtype."""
        x = self.hidden_states(input_ids, meta, k_cache, v_cache)
        if not (meta.is_decode and meta.logits_indices.shape[0] == x.shape[0]):
            x = x.index_select(0, meta.logits_indices)
        return mixers.stream_norm(x, self.W["ones"], self.W["norm"], self.cfg.norm_eps, self.dtype)

    def logits(self, hidden_last: torch.Tensor) -> torch.Tensor:
        lg = F.linear(hidden_last, self.W["lm_head"])
        return lg.float() * self.cfg.logit_scale if self.cfg.logit_scale != 1.0 else lg

    def sample(self, hidden_last: torch.Tensor, mask_bits: Optional[torch.Tensor],
               mask_idx: Optional[torch.Tensor]) -> torch.Tensor:
        """Greedy next tokens under the SAFE_DECODE mask: [S] int32 (a positive logit scale does not move the
        maximum, so the unscaled logits are compared)."""
        logits = F.linear(hidden_last, self.W["lm_head"])
        if self.cfg.logit_scale < 0:
            logits = -logits
        if logits.dtype == torch.bfloat16 and logits.shape[1] % 8 == 0 and logits.is_cuda:
            return ops.masked_argmax(logits, mask_bits, mask_idx)[0]
        return ops.ref.masked_argmax(logits, mask_bits, mask_idx)[0]
