"""Ops of the models that keep their residual stream in fp32 (`models/vivepel.py`): grouped RMS norm,
post-norm + layer scale + residual add, PolyNorm, per-head norm + partial rotary + cache append, and
attention with a chunked mask, soft-capped scores, a sink and head mixing.

Dispatch follows `ops/__init__.py`: a GPU tensor goes to the HIP kernel (`csrc/norms_f32.hip`,
`csrc/attention_chunk.hip`, built into `ops/lib/libkagent_mixers.so`) and raises if that library is
missing; a CPU tensor goes to the torch reference (`ops/reference.py`).  The activation dtype is bf16
or fp32; residual, norm weights, statistics, scores and weights are fp32 in both.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import reference as ref
from ._hip import check, require_mixers


TILE_MAX_BLOCKS = 4096   # block-table width the tile kernel stages in LDS (csrc/attention_chunk_tile.hip MAXPG)
TILE_MIN_Q = 8   # varlen steps whose longest row run is shorter stay on the per-token attention kernel


def _ref(t: torch.Tensor) -> bool:
    from . import _FORCE_REF
    return _FORCE_REF or not t.is_cuda


def _p(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def _stream() -> int:
    from . import _stream as s
    return s()


def _f32(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return 1
    if t.dtype == torch.bfloat16:
        return 0
    raise TypeError(f"activation dtype {t.dtype}: bf16 or fp32 expected")


def embed_f32(ids: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    """table[ids] as fp32 rows (the start of the residual stream)."""
    if _ref(table):
        return table[ids.long()].float()
    lib = require_mixers()
    T, (V, W) = ids.shape[0], table.shape
    out = torch.empty((T, W), dtype=torch.float32, device=table.device)
    assert ids.dtype == torch.int32 and table.is_contiguous()
    check(lib.ka_embed_f32(_p(out), _p(table), _p(ids), T, W, V, _f32(table), _stream()), "embed_f32")
    return out


def group_rmsnorm(x: torch.Tensor, w: torch.Tensor, groups: int, eps: float, out_dtype=None) -> torch.Tensor:
    out_dtype = out_dtype or x.dtype
    if _ref(x):
        return ref.group_rmsnorm(x, w, groups, eps, out_dtype)
    lib = require_mixers()
    rows, width = x.shape
    assert x.is_contiguous() and w.dtype == torch.float32 and w.shape[0] == width and width % groups == 0
    out = torch.empty((rows, width), dtype=out_dtype, device=x.device)
    check(lib.ka_group_rmsnorm(_p(out), _p(x), _p(w), rows, width, groups, float(eps), _f32(x), _f32(out), _stream()),
          "group_rmsnorm")
    return out


def post_norm_residual(resid: torch.Tensor, y: torch.Tensor, w_post: torch.Tensor, ls: torch.Tensor,
                       w_next: Optional[torch.Tensor], groups: int, eps: float) -> Optional[torch.Tensor]:
    """resid += ls * gnorm(y; w_post), in place; returns gnorm(resid; w_next) in y's dtype (None without w_next)."""
    if _ref(y):
        return ref.post_norm_residual(resid, y, w_post, ls, w_next, groups, eps)
    lib = require_mixers()
    rows, width = y.shape
    assert resid.dtype == torch.float32 and resid.shape == y.shape and resid.is_contiguous() and y.is_contiguous()
    assert w_post.dtype == torch.float32 and ls.dtype == torch.float32 and width % groups == 0
    assert w_post.shape[0] == width and ls.shape[0] == width and (w_next is None or w_next.shape[0] == width)
    out = torch.empty_like(y) if w_next is not None else None
    check(lib.ka_post_norm_residual(_p(resid), _p(y), _p(w_post), _p(ls), _p(w_next), _p(out), rows, width, groups,
                                    float(eps), _f32(y), _stream()), "post_norm_residual")
    return out


def polynorm(z: torch.Tensor, coef: torch.Tensor, eps: float) -> torch.Tensor:
    """coef[0] N(z) + coef[1] N(z^2) + coef[2] N(z^3) + coef[3] per row, N = divide by the row's rms."""
    if _ref(z):
        return ref.polynorm(z, coef, eps)
    lib = require_mixers()
    rows, ff = z.shape
    assert z.is_contiguous() and coef.dtype == torch.float32 and coef.numel() == 4
    out = torch.empty_like(z)
    check(lib.ka_polynorm(_p(out), _p(z), _p(coef), rows, ff, float(eps), _f32(z), _stream()), "polynorm")
    return out


def headnorm_rope_append(qk: torch.Tensor, q_w: torch.Tensor, k_w: torch.Tensor, inv_freq: torch.Tensor,
                         positions: torch.Tensor, slots: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                         H: int, G: int, D: int, rot: int, eps: float) -> torch.Tensor:
    """Fused [q | k] projection rows -> normed + rotated q [T, H, D]; the keys (normed + rotated) and
    the values (the keys as projected) are appended to the paged cache [NB, G, BS, D] at `slots`."""
    if _ref(qk):
        return ref.headnorm_rope_append(qk, q_w, k_w, inv_freq, positions, slots, k_cache, v_cache, H, G, D, rot, eps)
    lib = require_mixers()
    T = qk.shape[0]
    assert qk.is_contiguous() and qk.shape[1] == (H + G) * D and k_cache.dtype == qk.dtype == v_cache.dtype
    assert k_cache.shape[1:] == (G, k_cache.shape[2], D) and v_cache.shape == k_cache.shape
    assert positions.dtype == torch.int32 and slots.dtype == torch.int32 and inv_freq.numel() * 2 == rot
    assert positions.shape[0] >= T and slots.shape[0] >= T
    q = torch.empty((T, H, D), dtype=qk.dtype, device=qk.device)
    check(lib.ka_headnorm_rope_append(_p(q), _p(qk), _p(q_w), _p(k_w), _p(inv_freq), _p(positions), _p(slots),
                                      _p(k_cache), _p(v_cache), T, H, G, D, rot, float(eps), k_cache.shape[2],
                                      _f32(qk), _stream()), "headnorm_rope_append")
    return q


def chunk_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_tables: torch.Tensor,
                    q_starts: Optional[torch.Tensor], positions: torch.Tensor, slots: torch.Tensor,
                    mix: Optional[torch.Tensor], chunk: int, scale: float, cap: float, sink: bool,
                    max_q: int = 0, num_decode: int = 0) -> torch.Tensor:
    """q [T, H, D] -> [T, H * Dv].  q_starts [S + 1]: first row of each sequence in a varlen step (rows
    past q_starts[S] must be padding, slot < 0); None: token t is block-table row t (a decode step).  chunk 0: plain causal; cap 0: no soft cap; mix None: no head mixing."""
    if _ref(q):
        return ref.chunk_attention(q, k_cache, v_cache, block_tables, q_starts, positions, slots, mix, chunk, scale,
                                   cap, sink)
    lib = require_mixers()
    T, H, D = q.shape
    G, BS, Dv = k_cache.shape[1], k_cache.shape[2], v_cache.shape[3]
    assert q.is_contiguous() and k_cache.dtype == q.dtype == v_cache.dtype and k_cache.shape[3] == D
    assert block_tables.dtype == torch.int32 and block_tables.is_contiguous() and block_tables.dim() == 2
    assert positions.dtype == torch.int32 and slots.dtype == torch.int32
    assert q_starts is None or (q_starts.dtype == torch.int32 and q_starts.shape[0] == block_tables.shape[0] + 1)
    assert q_starts is not None or block_tables.shape[0] >= T
    assert mix is None or (mix.dtype == torch.float32 and mix.shape == (H, H) and mix.is_contiguous())
    if ((q_starts is None or max_q >= TILE_MIN_Q) and q.dtype == torch.bfloat16
            and block_tables.shape[1] <= TILE_MAX_BLOCKS and lib.ka_chunk_attention_tile_ok(H, G, D, Dv, BS)):
        # varlen: rows past the last sequence (a padded step) belong to no tile and stay zero;
        # decode (q_starts None): one workgroup per token writes every row
        varlen = q_starts is not None
        out = (torch.zeros if varlen else torch.empty)((T, H * Dv), dtype=q.dtype, device=q.device)
        tail = (H, G, D, Dv, int(chunk), BS, block_tables.shape[1], int(bool(sink)), float(scale), float(cap), _stream())
        nd = min(int(num_decode), block_tables.shape[0]) if varlen else 0
        if nd > 0:   # the leading one-token sequences: token t is block-table row t
            check(lib.ka_chunk_attention_tile(_p(out), _p(q), _p(k_cache), _p(v_cache), _p(block_tables), None, nd,
                                              _p(positions), _p(slots), _p(mix), 1, *tail), "chunk_attention_tile")
        S = block_tables.shape[0] - nd
        if not varlen:
            check(lib.ka_chunk_attention_tile(_p(out), _p(q), _p(k_cache), _p(v_cache), _p(block_tables), None, T,
                                              _p(positions), _p(slots), _p(mix), 1, *tail), "chunk_attention_tile")
        elif S > 0:   # (q_starts holds absolute rows, so the remaining sequences index q and out as they are)
            check(lib.ka_chunk_attention_tile(_p(out), _p(q), _p(k_cache), _p(v_cache), _p(block_tables[nd:]),
                                              _p(q_starts[nd:]), S, _p(positions), _p(slots), _p(mix), int(max_q), *tail),
                  "chunk_attention_tile")
        return out
    out = torch.empty((T, H * Dv), dtype=q.dtype, device=q.device)
    check(lib.ka_chunk_attention(_p(out), _p(q), _p(k_cache), _p(v_cache), _p(block_tables), _p(q_starts),
                                 block_tables.shape[0], _p(positions), _p(slots), _p(mix), T, H, G, D, Dv, int(chunk), BS,
                                 block_tables.shape[1], int(bool(sink)), float(scale), float(cap), _f32(q), _stream()),
          "chunk_attention")
    return out
