"""Ops of the models that keep their residual stream in fp32.  `models/vivepel.py`: grouped RMS norm,
post-norm + layer scale + residual add, PolyNorm, per-head norm + partial rotary + cache append, and
attention with a chunked mask, soft-capped scores, a sink and head mixing.  `models/kafilorn.py`: residual
streams (hyper-connections) with LayerNorm, the mLSTM gates and recurrence over state slots, latent attention
with a sliding window and a learned sink, squared ReLU, and expert routing in groups with a choice correction.
`models/suvapel.py`: Dynamic-Tanh norm and scaled residual sums, a gated token input, short convolutions over state
slots, rotary positions from a frequency table, sliding-window attention that keeps the first tokens with a per-head
gate, and the gated delta rule with a decay per head or per key channel.  `models/zibinex.py`: latent attention with
directly projected queries, interleaved rotary pairs and a per-head output gate, per-head norms before the cache
append, attention weights that are sigmoids of the score minus a logarithmic distance bias, a clamped gated unit, and
a sigmoid router whose weights scale the experts' inputs; each an option of the op it resembles.

Dispatch follows `ops/__init__.py`: a GPU tensor goes to the HIP kernel (the `csrc/*.hip` sources tagged
`KA_HIP_LIB: mixers`, built into `ops/lib/libkagent_mixers.so`) and raises if that library is
missing; a CPU tensor goes to the torch reference (`ops/reference.py`).  The activation dtype is bf16
or fp32; residual, norm weights, statistics, scores and weights are fp32 in both.
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn.functional as F

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


def post_norm_residual(resid: torch.Tensor, y: torch.Tensor, w_post: torch.Tensor, ls: Optional[torch.Tensor],
                       w_next: Optional[torch.Tensor], groups: int, eps: float, out_dtype=None) -> Optional[torch.Tensor]:
    """resid += ls * gnorm(y; w_post), in place (ls None: no layer scale); returns gnorm(resid; w_next) in out_dtype
    (default: y's dtype; y may be an fp32 sum in a bf16 engine), None without w_next."""
    out_dtype = out_dtype or y.dtype
    if _ref(y):
        return ref.post_norm_residual(resid, y, w_post, ls, w_next, groups, eps, out_dtype)
    lib = require_mixers()
    rows, width = y.shape
    assert resid.dtype == torch.float32 and resid.shape == y.shape and resid.is_contiguous() and y.is_contiguous()
    assert w_post.dtype == torch.float32 and (ls is None or ls.dtype == torch.float32) and width % groups == 0
    assert w_post.shape[0] == width and (ls is None or ls.shape[0] == width) and (w_next is None or w_next.shape[0] == width)
    out = torch.empty((rows, width), dtype=out_dtype, device=y.device) if w_next is not None else None
    check(lib.ka_post_norm_residual(_p(resid), _p(y), _p(w_post), _p(ls), _p(w_next), _p(out), rows, width, groups,
                                    float(eps), _f32(y), 1 if out_dtype == torch.float32 else 0, _stream()),
          "post_norm_residual")
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


# ------------------------------------------------------------------------------------------------
# residual streams, mLSTM, latent attention, grouped routing (csrc/streams_f32.hip, mlstm.hip,
# attention_latent.hip, moe_route.hip)
WINDOW_TILE = True   # bf16 window attention on the matrix cores where the shape allows (False: the per-token kernel)
MOE_GROUP_MAX = 1024  # bf16: token x expert rows served by the expert-grouped matrix-core kernels (decode steps)
MOE_ROWS_MAX = 64    # token x expert rows served by the matrix-vector expert kernels (decode steps); more: sorted GEMMs


def embed_streams(ids: torch.Tensor, table: torch.Tensor, scale: float, streams: int) -> torch.Tensor:
    """table[ids] * scale as fp32 in `streams` copies: the start of the residual streams [T, S, W]."""
    if _ref(table):
        return ref.embed_streams(ids, table, scale, streams)
    lib = require_mixers()
    T, (V, W) = ids.shape[0], table.shape
    assert ids.dtype == torch.int32 and table.is_contiguous() and streams >= 1
    out = torch.empty((T, streams, W), dtype=torch.float32, device=table.device)
    check(lib.ka_embed_streams(_p(out), _p(table), _p(ids), T, W, V, float(scale), streams, _f32(table), _stream()),
          "embed_streams")
    return out


def stream_norm(x: torch.Tensor, w_in: torch.Tensor, w: torch.Tensor, eps: float, out_dtype) -> torch.Tensor:
    """LayerNorm (weight, no bias) of sum_s w_in[s] x[:, s]: [T, S, W] fp32 -> [T, W] in out_dtype."""
    if _ref(x):
        return ref.stream_norm(x, w_in, w, eps, out_dtype)
    lib = require_mixers()
    T, S, W = x.shape
    assert x.dtype == torch.float32 and x.is_contiguous() and w_in.dtype == torch.float32 and w_in.numel() == S
    assert w.dtype == torch.float32 and w.numel() == W
    out = torch.empty((T, W), dtype=out_dtype, device=x.device)
    check(lib.ka_stream_norm(_p(out), _p(x), _p(w_in), _p(w), T, W, S, float(eps), _f32(out), _stream()), "stream_norm")
    return out


def stream_update(x: torch.Tensor, y: torch.Tensor, mix: torch.Tensor, out: torch.Tensor,
                  next_in: Optional[torch.Tensor], next_w: Optional[torch.Tensor], eps: float, out_dtype):
    """x[:, r] <- sum_s mix[s, r] x[:, s] + out[r] * y, in place; returns stream_norm(x, next_in, next_w) computed
    in the same pass (None without next_w)."""
    if _ref(x):
        return ref.stream_update(x, y, mix, out, next_in, next_w, eps, out_dtype)
    lib = require_mixers()
    T, S, W = x.shape
    assert x.dtype == torch.float32 and x.is_contiguous() and y.shape == (T, W) and y.is_contiguous()
    assert mix.dtype == torch.float32 and mix.shape == (S, S) and mix.is_contiguous() and out.dtype == torch.float32
    assert out.numel() == S and (next_w is None or (next_w.dtype == torch.float32 and next_w.numel() == W
                                                     and next_in.dtype == torch.float32 and next_in.numel() == S))
    h = torch.empty((T, W), dtype=out_dtype, device=x.device) if next_w is not None else None
    check(lib.ka_stream_update(_p(x), _p(y), _p(mix), _p(out), _p(next_in) if next_w is not None else None, _p(next_w),
                               _p(h), T, W, S, float(eps), _f32(y), _f32(h) if h is not None else 0, _stream()),
          "stream_update")
    return h


def relu_sq(z: torch.Tensor) -> torch.Tensor:
    """relu(z)^2, elementwise."""
    if _ref(z):
        return ref.relu_sq(z)
    lib = require_mixers()
    assert z.is_contiguous()
    out = torch.empty_like(z)
    check(lib.ka_relu_sq(_p(out), _p(z), z.numel(), _f32(z), _stream()), "relu_sq")
    return out


def silu_mul(gu: torch.Tensor, row_scale: Optional[torch.Tensor] = None) -> torch.Tensor:
    """[T, 2 ff] = gate | up -> silu(gate) * up [T, ff] (bf16 or fp32).  row_scale [T] fp32: the rows' inputs were
    to be multiplied by these numbers before the two projections; as those are linear, silu(s gate) * (s up)."""
    if _ref(gu):
        return ref.silu_mul(gu) if row_scale is None else ref.silu_mul_scaled(gu, row_scale)
    lib = require_mixers()
    T, two = gu.shape
    assert gu.is_contiguous() and two % 2 == 0
    assert row_scale is None or (row_scale.dtype == torch.float32 and row_scale.shape == (T,) and row_scale.is_contiguous())
    out = torch.empty((T, two // 2), dtype=gu.dtype, device=gu.device)
    check(lib.ka_silu_mul_rows(_p(out), _p(gu), _p(row_scale), T, two // 2, _f32(gu), _stream()), "silu_mul_rows")
    return out


def glu_clamp(gu: torch.Tensor, limit: float, alpha: float) -> torch.Tensor:
    """[T, 2 ff] = gate | up -> g sigmoid(alpha g) (u + 1) [T, ff] with g = min(gate, limit) and
    u = clamp(up, -limit, limit)."""
    if _ref(gu):
        return ref.glu_clamp(gu, limit, alpha)
    lib = require_mixers()
    T, two = gu.shape
    assert gu.is_contiguous() and two % 2 == 0
    out = torch.empty((T, two // 2), dtype=gu.dtype, device=gu.device)
    check(lib.ka_glu_clamp(_p(out), _p(gu), T, two // 2, float(limit), float(alpha), _f32(gu), _stream()), "glu_clamp")
    return out


def mlstm_gates(h: torch.Tensor, w_if: torch.Tensor, b_if: torch.Tensor, cap: float,
                w_lp: Optional[torch.Tensor] = None) -> torch.Tensor:
    """[T, 2H] fp32: log input gates (soft-capped), then log forget gates logsigmoid(soft-capped).  w_lp: a bf16
    copy of w_if holding the same values (weights that a checkpoint stores in bf16): bf16 rows then run on the
    matrix cores, where products of bf16 inputs are exact and accumulate in fp32."""
    if _ref(h):
        return ref.mlstm_gates(h, w_if, b_if, cap)
    lib = require_mixers()
    T, W = h.shape
    if (w_lp is not None and h.dtype == torch.bfloat16 and w_lp.dtype == torch.bfloat16 and W % 128 == 0
            and w_lp.shape[0] <= 128):
        assert h.is_contiguous() and w_lp.is_contiguous() and w_lp.shape == w_if.shape and b_if.dtype == torch.float32
        out = torch.empty((T, w_lp.shape[0]), dtype=torch.float32, device=h.device)
        check(lib.ka_mlstm_gates_mfma(_p(out), _p(h), _p(w_lp), _p(b_if), T, W, w_lp.shape[0] // 2, float(cap), _stream()),
              "mlstm_gates_mfma")
        return out
    assert h.is_contiguous() and w_if.dtype == torch.float32 and w_if.shape[1] == W and w_if.is_contiguous()
    assert b_if.dtype == torch.float32 and b_if.numel() == w_if.shape[0] and w_if.shape[0] % 2 == 0
    out = torch.empty((T, w_if.shape[0]), dtype=torch.float32, device=h.device)
    check(lib.ka_mlstm_gates(_p(out), _p(h), _p(w_if), _p(b_if), T, W, w_if.shape[0] // 2, float(cap), _f32(h), _stream()),
          "mlstm_gates")
    return out


def mlstm_scan(proj: torch.Tensor, q_off: int, k_off: int, v_off: int, gates: torch.Tensor, st_S: torch.Tensor,
               st_n: torch.Tensor, st_m: torch.Tensor, seq_slots: torch.Tensor, q_starts: Optional[torch.Tensor],
               positions: torch.Tensor, H: int, D: int, Dv: int, qscale: float) -> torch.Tensor:
    """The mLSTM recurrence over each sequence's rows, from / into the state of its slot (st_S [slots, H, Dv, D],
    st_n [slots, H, D], st_m [slots, H], fp32); a sequence whose first row is at position 0 starts from zero.
    q_starts None: row t is sequence t.  -> (numerators S^T q [T, H * Dv], denominators max(|n . q|, exp(-m)) + 1e-6
    [T, H]), fp32; `headnorm_gate` divides."""
    if _ref(proj):
        S = st_S.transpose(-1, -2)
        return ref.mlstm_scan(proj, q_off, k_off, v_off, gates, S, st_n, st_m, seq_slots, q_starts, positions, H, D, Dv,
                              qscale)
    lib = require_mixers()
    T, P = proj.shape
    nseq = seq_slots.shape[0]
    assert proj.is_contiguous() and gates.dtype == torch.float32 and gates.shape == (T, 2 * H) and gates.is_contiguous()
    assert max(q_off, k_off) + H * D <= P and v_off + H * Dv <= P
    assert st_S.dtype == st_n.dtype == st_m.dtype == torch.float32 and st_S.shape[1:] == (H, Dv, D) and st_S.is_contiguous()
    assert st_n.shape[1:] == (H, D) and st_m.shape[1:] == (H,) and st_n.is_contiguous() and st_m.is_contiguous()
    assert seq_slots.dtype == torch.int32 and positions.dtype == torch.int32 and positions.shape[0] >= T
    assert (q_starts is None and nseq <= T) or (q_starts is not None and q_starts.dtype == torch.int32
                                                 and q_starts.shape[0] == nseq + 1)
    out = torch.zeros((T, H * Dv), dtype=torch.float32, device=proj.device)
    den = torch.ones((T, H), dtype=torch.float32, device=proj.device)
    dec = torch.empty((T, H, 3), dtype=torch.float32, device=proj.device)   # per row: forget factor, input factor, exp(-max)
    check(lib.ka_mlstm_scan(_p(out), _p(den), _p(proj), P, q_off, k_off, v_off, _p(gates), _p(dec), _p(st_S), _p(st_n),
                            _p(st_m), _p(seq_slots), _p(q_starts), nseq, _p(positions), H, D, Dv, float(qscale), _f32(proj),
                            _stream()), "mlstm_scan")
    return out, den


def headnorm_gate(o: torch.Tensor, proj: torch.Tensor, g_off: int, w: torch.Tensor, H: int, Dv: int, eps: float,
                  out_dtype, den: Optional[torch.Tensor] = None, silu: bool = False) -> torch.Tensor:
    """o [T, H * Dv] fp32 (each head first divided by den [T, H], if given): each head divided by its root mean
    square, times w, times sigmoid(proj[:, g_off:...]) (silu: times silu of those columns)."""
    if _ref(o):
        return ref.headnorm_gate(o, proj, g_off, w, H, Dv, eps, out_dtype, den, silu)
    lib = require_mixers()
    T = o.shape[0]
    assert o.dtype == torch.float32 and o.is_contiguous() and proj.is_contiguous() and proj.dtype == out_dtype
    assert g_off + H * Dv <= proj.shape[1] and w.dtype == torch.float32 and w.numel() == H * Dv
    assert den is None or (den.dtype == torch.float32 and den.shape == (T, H) and den.is_contiguous())
    out = torch.empty((T, H * Dv), dtype=out_dtype, device=o.device)
    check(lib.ka_headnorm_gate(_p(out), _p(o), _p(den), _p(proj), proj.shape[1], g_off, _p(w), T, H, Dv, float(eps),
                               int(bool(silu)), _f32(out), _stream()), "headnorm_gate")
    return out


def latent_prep(proj: torch.Tensor, Q: int, R: int, Dr: int, w_q: Optional[torch.Tensor], w_kv: Optional[torch.Tensor],
                inv_freq: torch.Tensor, positions: torch.Tensor, slots: torch.Tensor, cache: Optional[torch.Tensor],
                rot_dims: int, eps: float, interleaved: bool = False, mag: float = 1.0) -> Optional[torch.Tensor]:
    """Rows [query latent Q | key/value latent R | rotated key part Dr] -> the RMS-normed query latent [T, Q] (Q = 0,
    a model that projects its queries directly: None); with a cache [NB, BS, R + Dr], the normed latent and the
    rotated key part are appended at `slots`.  Rotary pairs are (i, i + rot_dims / 2), or (2i, 2i + 1) when
    interleaved; cos and sin are multiplied by `mag`."""
    if _ref(proj):
        return ref.latent_prep(proj, Q, R, Dr, w_q, w_kv, inv_freq, positions, slots, cache, rot_dims, eps, interleaved, mag)
    lib = require_mixers()
    T, P = proj.shape
    assert proj.is_contiguous() and (Q == 0 or (w_q.dtype == torch.float32 and w_q.numel() == Q))
    assert positions.dtype == torch.int32 and slots.dtype == torch.int32 and positions.shape[0] >= T and slots.shape[0] >= T
    if cache is not None:
        assert cache.dtype == proj.dtype and cache.shape[2] == R + Dr and cache.is_contiguous() and P >= Q + R + Dr
        assert w_kv.dtype == torch.float32 and w_kv.numel() == R and inv_freq.dtype == torch.float32
        assert inv_freq.numel() * 2 == rot_dims
    cq = torch.empty((T, Q), dtype=proj.dtype, device=proj.device) if Q else None
    check(lib.ka_latent_prep(_p(cq), _p(proj), T, P, Q, R, Dr, _p(w_q), _p(w_kv), _p(inv_freq), _p(positions), _p(slots),
                             _p(cache), rot_dims, float(eps), int(bool(interleaved)), float(mag), _f32(proj), _stream()),
          "latent_prep")
    return cq


def rope_split_q(q: torch.Tensor, inv_freq: torch.Tensor, positions: torch.Tensor, H: int, D: int, Dr: int,
                 rot_dims: int, interleaved: bool = False, mag: float = 1.0, off: int = 0):
    """The columns off .. off + H * (D + Dr) of q's rows (q may be a fused projection) -> (unrotated parts [H, T, D]
    in q's dtype, rotated parts after rotary [T, H, Dr] fp32).  Rotary as in `latent_prep`."""
    if _ref(q):
        return ref.rope_split_q(q, inv_freq, positions, H, D, Dr, rot_dims, interleaved, mag, off)
    lib = require_mixers()
    T, P = q.shape
    assert q.is_contiguous() and 0 <= off and off + H * (D + Dr) <= P and positions.dtype == torch.int32
    assert positions.shape[0] >= T and (rot_dims == 0 or (inv_freq.dtype == torch.float32 and inv_freq.numel() * 2 == rot_dims))
    qn = torch.empty((H, T, D), dtype=q.dtype, device=q.device)
    qr = torch.empty((T, H, Dr), dtype=torch.float32, device=q.device)
    check(lib.ka_rope_split_q(_p(qn), _p(qr), _p(q), P, off, _p(inv_freq), _p(positions), T, H, D, Dr, rot_dims,
                              int(bool(interleaved)), float(mag), _f32(q), _stream()), "rope_split_q")
    return qn, qr


def head_gate(o: torch.Tensor, gate_src: Optional[torch.Tensor], g_off: int = 0) -> torch.Tensor:
    """o [H, T, Dv] (a batched per-head product) -> [T, H * Dv], head h times sigmoid(gate_src[t, g_off + h])
    (gate_src None: the layout change only)."""
    if _ref(o):
        return ref.head_gate(o, gate_src, g_off)
    lib = require_mixers()
    H, T, Dv = o.shape
    assert o.is_contiguous()
    gs = 0
    if gate_src is not None:
        assert gate_src.dtype == o.dtype and gate_src.is_contiguous() and gate_src.shape[0] >= T
        gs = gate_src.shape[1]
        assert 0 <= g_off and g_off + H <= gs
    out = torch.empty((T, H * Dv), dtype=o.dtype, device=o.device)
    check(lib.ka_head_gate(_p(out), _p(o), _p(gate_src), gs, g_off, T, H, Dv, _f32(o), _stream()), "head_gate")
    return out


def window_attention(q_lat: torch.Tensor, q_rot: torch.Tensor, cache: torch.Tensor, block_tables: torch.Tensor,
                     q_starts: Optional[torch.Tensor], positions: torch.Tensor, slots: torch.Tensor,
                     sink: Optional[torch.Tensor], window: int, scale: float) -> torch.Tensor:
    """Multi-query attention over cache rows [latent R | rotated key part Dr] with the latent as the value:
    q_lat [H, T, R], q_rot [T, H, Dr] fp32 -> [H, T, R].  window 0: all earlier keys; sink None: plain softmax."""
    if _ref(q_lat):
        return ref.window_attention(q_lat, q_rot, cache, block_tables, q_starts, positions, slots, sink, window, scale)
    lib = require_mixers()
    H, T, R = q_lat.shape
    Dr, BS = q_rot.shape[2], cache.shape[1]
    assert q_lat.is_contiguous() and q_rot.is_contiguous() and q_rot.dtype == torch.float32 and q_rot.shape[:2] == (T, H)
    assert cache.dtype == q_lat.dtype and cache.is_contiguous() and cache.shape[2] == R + Dr
    assert block_tables.dtype == torch.int32 and block_tables.is_contiguous() and block_tables.dim() == 2
    assert positions.dtype == torch.int32 and slots.dtype == torch.int32 and positions.shape[0] >= T and slots.shape[0] >= T
    assert q_starts is None or (q_starts.dtype == torch.int32 and q_starts.shape[0] == block_tables.shape[0] + 1)
    assert q_starts is not None or block_tables.shape[0] >= T
    assert sink is None or (sink.dtype == torch.float32 and sink.numel() == H)
    out = torch.empty((H, T, R), dtype=q_lat.dtype, device=q_lat.device)
    check(lib.ka_window_attention(_p(out), _p(q_lat), _p(q_rot), _p(cache), _p(block_tables), _p(q_starts),
                                  block_tables.shape[0], _p(positions), _p(slots), _p(sink), T, H, R, Dr, BS,
                                  block_tables.shape[1], int(window), float(scale), _f32(q_lat),
                                  0 if WINDOW_TILE else 1, _stream()),
          "window_attention")
    return out


def moe_route(h: torch.Tensor, w_router: torch.Tensor, correction: Optional[torch.Tensor], top: int, groups: int,
              keep: int, sigmoid: bool = False, renorm: bool = True):
    """-> (expert ids [T, top] int32, weights [T, top] fp32); see csrc/moe_route.hip.  sigmoid: the scores are the
    logits' sigmoids instead of their softmax; renorm False: the weights are the chosen scores as they are."""
    if _ref(h):
        return ref.moe_route(h, w_router, correction, top, groups, keep, sigmoid, renorm)
    lib = require_mixers()
    T, W = h.shape
    E = w_router.shape[0]
    assert h.is_contiguous() and w_router.dtype == torch.float32 and w_router.shape[1] == W and w_router.is_contiguous()
    assert correction is None or (correction.dtype == torch.float32 and correction.numel() == E)
    ids = torch.empty((T, top), dtype=torch.int32, device=h.device)
    w = torch.empty((T, top), dtype=torch.float32, device=h.device)
    check(lib.ka_moe_route(_p(ids), _p(w), _p(h), _p(w_router), _p(correction), T, W, E, top, groups, keep,
                           int(bool(sigmoid)), int(bool(renorm)), _f32(h), _stream()), "moe_route")
    return ids, w


def moe_experts(h: torch.Tensor, w_gu: torch.Tensor, w_down: torch.Tensor, ids: torch.Tensor, w: torch.Tensor,
                scale_input: bool = False) -> torch.Tensor:
    """sum_k w[t, k] * expert_{ids[t, k]}(h[t]) -> [T, W] fp32; w_gu [E, 2 ff, W] (gate rows, then up rows),
    w_down [E, W, ff].  scale_input: sum_k expert_{ids[t, k]}(w[t, k] * h[t]) instead (the weight enters before the
    expert's nonlinearity; it is applied to the fp32 results of the gate and up projections, which are linear).  Decode-sized steps: in bf16 the rows grouped by expert on the matrix cores, otherwise
    matrix-vector kernels straight from the stacked weights; neither reads the host, both are capturable.  More: rows sorted by expert, one read of the per-expert counts, one vendor GEMM pair per
    expert segment, weighted scatter-add in fp32."""
    if _ref(h):
        return ref.moe_experts(h, w_gu, w_down, ids, w, scale_input)
    T, W = h.shape
    E, two_ff, _ = w_gu.shape
    ff, top = two_ff // 2, ids.shape[1]
    assert h.is_contiguous() and w_gu.is_contiguous() and w_down.is_contiguous() and w_gu.dtype == h.dtype == w_down.dtype
    assert w_down.shape == (E, W, ff) and ids.dtype == torch.int32 and w.dtype == torch.float32 and w.shape == ids.shape
    out = torch.zeros((T, W), dtype=torch.float32, device=h.device)
    if h.dtype == torch.bfloat16 and T * top <= MOE_GROUP_MAX and W % 32 == 0 and ff % 32 == 0:
        lib = require_mixers()   # rows grouped by expert on the matrix cores: every expert's weights read once
        act = torch.empty((T * top, ff), dtype=h.dtype, device=h.device)
        yk = torch.empty((T * top, W), dtype=torch.float32, device=h.device)
        check(lib.ka_moe_grouped(_p(out), _p(act), _p(yk), _p(h), _p(w_gu), _p(w_down), _p(ids), _p(w), T, W, ff, top, E,
                                 int(bool(scale_input)), _stream()), "moe_grouped")
        return out
    rows_ok = W * 4 <= 60 * 1024 and top * ff * 4 <= 60 * 1024 and top <= 32
    capturing = torch.cuda.is_current_stream_capturing()     # a graph cannot hold the sorted path's host read
    if capturing and not rows_ok:
        raise RuntimeError(f"moe_experts: width {W} / top {top} x ff {ff} outside the capturable kernels' limits")
    if rows_ok and (capturing or T * top <= MOE_ROWS_MAX):
        lib = require_mixers()
        act = torch.empty((T * top, ff), dtype=h.dtype, device=h.device)
        check(lib.ka_moe_rows(_p(out), _p(act), _p(h), _p(w_gu), _p(w_down), _p(ids), _p(w), T, W, ff, top,
                              int(bool(scale_input)), _f32(h), _stream()), "moe_rows")
        return out
    flat = ids.reshape(-1).long()
    order = torch.argsort(flat, stable=True)
    counts = torch.bincount(flat, minlength=E).tolist()    # the layer's one host read (vendor GEMMs take host shapes)
    tok = torch.div(order, top, rounding_mode="floor")
    xs = h.index_select(0, tok)
    ys = torch.empty((xs.shape[0], W), dtype=h.dtype, device=h.device)
    ws = w.reshape(-1).index_select(0, order).contiguous()
    off = 0
    for e, c in enumerate(counts):
        if c:
            gu = F.linear(xs[off:off + c], w_gu[e])
            ys[off:off + c] = F.linear(silu_mul(gu, ws[off:off + c] if scale_input else None), w_down[e])
            off += c
    out.index_add_(0, tok, ys.float() if scale_input else ys.float() * ws.unsqueeze(1))
    return out


# ------------------------------------------------------------------------------------------------
# Dynamic-Tanh norm and scaled residual sums (csrc/residual_dyt.hip), short convolutions over state slots
# (csrc/short_conv.hip), rotary positions from a frequency table + sliding-window attention that keeps the first
# tokens (csrc/attention_window.hip), the gated delta rule (csrc/delta_rule.hip)
def _dyt_ok(dyt, width: int) -> None:
    alpha, w, b = dyt
    assert alpha.dtype == w.dtype == b.dtype == torch.float32 and alpha.numel() == 1 and w.numel() == b.numel() == width


def dyt_norm(x: torch.Tensor, alpha: torch.Tensor, w: torch.Tensor, b: torch.Tensor, out_dtype) -> torch.Tensor:
    """Dynamic Tanh: tanh(alpha * x) * w + b per entry, no statistics.  x [T, W] fp32, alpha a one-element fp32
    tensor -> [T, W] in out_dtype."""
    if _ref(x):
        return ref.dyt_norm(x, alpha, w, b, out_dtype)
    lib = require_mixers()
    T, W = x.shape
    assert x.dtype == torch.float32 and x.is_contiguous()
    _dyt_ok((alpha, w, b), W)
    out = torch.empty((T, W), dtype=out_dtype, device=x.device)
    check(lib.ka_dyt_norm(_p(out), _p(x), _p(alpha), _p(w), _p(b), T, W, _f32(out), _stream()), "dyt_norm")
    return out


def residual_mix(x: torch.Tensor, ys, coefs, out_dtype, want_copy: bool = False, dyt=None):
    """x [T, W] fp32 += sum_i coefs[i] * ys[i] in place (one to three sublayer results in the activation dtype,
    summed in fp32); returns (x rounded to out_dtype if want_copy, dyt_norm(x, *dyt) if dyt = (alpha, w, b)), both
    written in the same pass."""
    assert 1 <= len(ys) <= 3 and len(ys) == len(coefs)
    if _ref(x):
        return ref.residual_mix(x, ys, coefs, out_dtype, want_copy, dyt)
    lib = require_mixers()
    T, W = x.shape
    assert x.dtype == torch.float32 and x.is_contiguous()
    for y in ys:
        assert y.shape == (T, W) and y.is_contiguous() and y.dtype == ys[0].dtype
    if dyt is not None:
        _dyt_ok(dyt, W)
    yp = [_p(y) for y in ys] + [None] * (3 - len(ys))
    cs = [float(c) for c in coefs] + [0.0] * (3 - len(ys))
    xa = torch.empty((T, W), dtype=out_dtype, device=x.device) if want_copy else None
    h = torch.empty((T, W), dtype=out_dtype, device=x.device) if dyt is not None else None
    al, dw, db = dyt if dyt is not None else (None, None, None)
    check(lib.ka_residual_mix(_p(x), *yp, *cs, _p(xa), _p(h), _p(al), _p(dw), _p(db), T, W, _f32(ys[0]),
                              1 if out_dtype == torch.float32 else 0, _stream()), "residual_mix")
    return xa, h


def rms_residual(x: torch.Tensor, y: torch.Tensor, w: torch.Tensor, mult: float, eps: float, out_dtype, dyt=None):
    """x [T, W] fp32 += mult * y / sqrt(mean(y^2) + eps) * w in place; returns dyt_norm(x, *dyt) from the same pass
    (None without dyt)."""
    if _ref(x):
        return ref.rms_residual(x, y, w, mult, eps, out_dtype, dyt)
    lib = require_mixers()
    T, W = x.shape
    assert x.dtype == torch.float32 and x.is_contiguous() and y.shape == (T, W) and y.is_contiguous()
    assert w.dtype == torch.float32 and w.numel() == W
    if dyt is not None:
        _dyt_ok(dyt, W)
    h = torch.empty((T, W), dtype=out_dtype, device=x.device) if dyt is not None else None
    al, dw, db = dyt if dyt is not None else (None, None, None)
    check(lib.ka_rms_residual(_p(x), _p(y), _p(w), float(mult), float(eps), _p(h), _p(al), _p(dw), _p(db), T, W, _f32(y),
                              1 if out_dtype == torch.float32 else 0, _stream()), "rms_residual")
    return h


def gelu_gate_embed(z: torch.Tensor, table: torch.Tensor, ids: torch.Tensor, col0: int) -> torch.Tensor:
    """gelu_tanh(z) * table[ids, col0 : col0 + dim] for z [T, dim]: a gate on a slice of an embedding row."""
    if _ref(z):
        return ref.gelu_gate_embed(z, table, ids, col0)
    lib = require_mixers()
    T, dim = z.shape
    assert z.is_contiguous() and table.is_contiguous() and table.dtype == z.dtype and ids.dtype == torch.int32
    assert 0 <= col0 and col0 + dim <= table.shape[1] and ids.shape[0] >= T
    out = torch.empty_like(z)
    check(lib.ka_gelu_gate_embed(_p(out), _p(z), _p(table), _p(ids), T, dim, table.shape[1], col0, table.shape[0], _f32(z),
                                 _stream()), "gelu_gate_embed")
    return out


def silu_mul_bias(proj: torch.Tensor, off: int, ff: int, bias: torch.Tensor) -> torch.Tensor:
    """silu(gate + bias[:ff]) * (up + bias[ff:]) with gate | up = proj[:, off : off + 2 ff] -> [T, ff]."""
    if _ref(proj):
        return ref.silu_mul_bias(proj, off, ff, bias)
    lib = require_mixers()
    T, P = proj.shape
    assert proj.is_contiguous() and off >= 0 and off + 2 * ff <= P and bias.dtype == torch.float32 and bias.numel() == 2 * ff
    out = torch.empty((T, ff), dtype=proj.dtype, device=proj.device)
    check(lib.ka_silu_mul_bias(_p(out), _p(proj), P, off, ff, _p(bias), T, _f32(proj), _stream()), "silu_mul_bias")
    return out


def short_conv(proj: torch.Tensor, off: int, C: int, w: torch.Tensor, state: Optional[torch.Tensor],
               seq_slots: torch.Tensor, q_starts: Optional[torch.Tensor], positions: torch.Tensor, act: bool) -> torch.Tensor:
    """A causal convolution over time per channel, y_t = sum_j w[j] * u_(t - taps + 1 + j), on the columns
    u = proj[:, off : off + C] of each sequence's rows.  Inputs from before this step come from state[slot]
    [taps - 1, C] (the sequence's last inputs, newest last), inputs before position 0 are zero, so a slot needs no
    clearing; afterwards the state holds the last inputs including this step's.  act: silu on the result.
    w [taps, C] fp32 (tap-major: w[j] meets the row taps - 1 - j back); state [slots, taps - 1, C] in proj's dtype
    (None when taps is 1).  q_starts None: row t is sequence t.  -> [T, C]."""
    taps = w.shape[0]
    if _ref(proj):
        return ref.short_conv(proj, off, C, w, state, seq_slots, q_starts, positions, act)
    lib = require_mixers()
    T, P = proj.shape
    nseq = seq_slots.shape[0]
    assert proj.is_contiguous() and off >= 0 and off + C <= P and w.dtype == torch.float32 and w.shape == (taps, C)
    assert w.is_contiguous() and seq_slots.dtype == torch.int32 and positions.dtype == torch.int32 and positions.shape[0] >= T
    assert taps == 1 or (state is not None and state.dtype == proj.dtype and state.shape[1:] == (taps - 1, C)
                         and state.is_contiguous())
    assert (q_starts is None and nseq <= T) or (q_starts is not None and q_starts.dtype == torch.int32
                                                 and q_starts.shape[0] == nseq + 1)
    out = torch.zeros((T, C), dtype=proj.dtype, device=proj.device)
    check(lib.ka_short_conv(_p(out), _p(proj), P, off, C, _p(w), taps, _p(state), _p(seq_slots), _p(q_starts), nseq,
                            _p(positions), T, int(bool(act)), _f32(proj), _stream()), "short_conv")
    return out


def rope_append(qkv: torch.Tensor, inv_freq: Optional[torch.Tensor], mag: float, positions: torch.Tensor,
                slots: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, H: int, G: int, D: int, Dv: int,
                rot: int, q_norm: Optional[torch.Tensor] = None, k_norm: Optional[torch.Tensor] = None,
                eps: float = 0.0) -> torch.Tensor:
    """Rows [q (H x D) | k (G x D) | v (G x Dv)] -> q [T, H, D]; with q_norm / k_norm [D] fp32 every q / k head is
    first divided by its root mean square (eps inside the root) and multiplied by that weight; then rotary positions on the first `rot` entries of
    each head (pairs (i, i + rot/2), angle = position * inv_freq[i] in fp32, cos and sin times `mag`); the rotated
    keys and the values are appended to the paged cache [NB, G, BS, D] / [NB, G, Dv, BS] at `slots` (-1: skipped)."""
    if _ref(qkv):
        return ref.rope_append(qkv, inv_freq, mag, positions, slots, k_cache, v_cache, H, G, D, Dv, rot, q_norm, k_norm, eps)
    lib = require_mixers()
    T = qkv.shape[0]
    assert qkv.is_contiguous() and qkv.shape[1] == (H + G) * D + G * Dv and k_cache.dtype == qkv.dtype == v_cache.dtype
    assert k_cache.shape[1:] == (G, k_cache.shape[2], D) and v_cache.shape == (k_cache.shape[0], G, Dv, k_cache.shape[2])
    assert k_cache.is_contiguous() and v_cache.is_contiguous()
    assert positions.dtype == torch.int32 and slots.dtype == torch.int32 and positions.shape[0] >= T and slots.shape[0] >= T
    assert rot == 0 or (inv_freq.dtype == torch.float32 and inv_freq.numel() * 2 == rot and rot <= D)
    for nw in (q_norm, k_norm):
        assert nw is None or (nw.dtype == torch.float32 and nw.numel() == D and nw.is_contiguous())
    q = torch.empty((T, H, D), dtype=qkv.dtype, device=qkv.device)
    check(lib.ka_rope_append(_p(q), _p(qkv), _p(inv_freq), float(mag), _p(positions), _p(slots), _p(k_cache), _p(v_cache),
                             T, H, G, D, Dv, rot, k_cache.shape[2], _p(q_norm), _p(k_norm), float(eps), _f32(qkv), _stream()),
          "rope_append")
    return q


SLIDING_TILE = True   # bf16 prompt portions of sliding attention on the matrix cores where the shape allows


def sliding_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_tables: torch.Tensor,
                      q_starts: Optional[torch.Tensor], positions: torch.Tensor, slots: torch.Tensor,
                      gate_src: Optional[torch.Tensor], g_off: int, window: int, keep_first: int, scale: float,
                      max_q: int = 0, num_decode: int = 0, dist: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Softmax attention with grouped keys / values over a paged cache (k_cache [NB, G, BS, D], v_cache
    [NB, G, Dv, BS]): the query at position p sees the keys j <= p with p - j < window or j < keep_first (window 0:
    all of 0 .. p; kept keys stay at their own positions).  Head h's result is multiplied by
    sigmoid(gate_src[t, g_off + h]) (gate_src None: no gate).  q [T, H, D] -> [T, H * Dv].
    q_starts None: row t is block-table row t (a decode step).  max_q: the longest run of rows of one sequence in a
    varlen step (0: unknown), num_decode: its leading one-row sequences; they choose the kernel, not the result.
    dist [3, H] fp32 = (r1, r2, pb) per head: no softmax; the weight of a visible key at distance p - j is
    sigmoid(score - r1 ln(1 + r2 (p - j)) + pb), and the weights are not normalised over the keys."""
    if _ref(q):
        return ref.sliding_attention(q, k_cache, v_cache, block_tables, q_starts, positions, slots, gate_src, g_off,
                                     window, keep_first, scale, dist)
    lib = require_mixers()
    T, H, D = q.shape
    G, BS, Dv = k_cache.shape[1], k_cache.shape[2], v_cache.shape[2]
    assert q.is_contiguous() and k_cache.dtype == q.dtype == v_cache.dtype and k_cache.shape[3] == D and H % G == 0
    assert v_cache.shape == (k_cache.shape[0], G, Dv, BS) and k_cache.is_contiguous() and v_cache.is_contiguous()
    assert block_tables.dtype == torch.int32 and block_tables.is_contiguous() and block_tables.dim() == 2
    assert positions.dtype == torch.int32 and slots.dtype == torch.int32 and positions.shape[0] >= T and slots.shape[0] >= T
    assert q_starts is None or (q_starts.dtype == torch.int32 and q_starts.shape[0] == block_tables.shape[0] + 1)
    assert q_starts is not None or block_tables.shape[0] >= T
    gs = 0
    if gate_src is not None:
        assert gate_src.dtype == q.dtype and gate_src.is_contiguous() and gate_src.shape[0] >= T
        gs = gate_src.shape[1]
        assert 0 <= g_off and g_off + H <= gs
    assert dist is None or (dist.dtype == torch.float32 and dist.shape == (3, H) and dist.is_contiguous())

    def tail(rows):
        return (_p(positions), _p(slots), _p(gate_src), gs, g_off, rows, H, G, D, Dv, int(window), int(keep_first), BS,
                block_tables.shape[1], float(scale), _p(dist), _f32(q))

    tile = SLIDING_TILE and q.dtype == torch.bfloat16 and lib.ka_sliding_attention_tile_ok(H, G, D, Dv, BS)
    if tile and q_starts is not None and max_q >= 8:
        # rows past the last sequence (a padded step) belong to no tile and stay zero
        out = torch.zeros((T, H * Dv), dtype=q.dtype, device=q.device)
        nd = min(int(num_decode), block_tables.shape[0])
        if nd > 0:   # the leading one-row sequences: rows 0 .. nd - 1 only, row t is block-table row t
            check(lib.ka_sliding_attention(_p(out), _p(q), _p(k_cache), _p(v_cache), _p(block_tables), None, nd, *tail(nd), 1,
                                           _stream()), "sliding_attention")
        if block_tables.shape[0] > nd:   # (q_starts holds absolute rows, so the remaining sequences index q and out as they are)
            check(lib.ka_sliding_attention(_p(out), _p(q), _p(k_cache), _p(v_cache), _p(block_tables[nd:]), _p(q_starts[nd:]),
                                           block_tables.shape[0] - nd, *tail(T), int(max_q), _stream()), "sliding_attention_tile")
        return out
    out = torch.empty((T, H * Dv), dtype=q.dtype, device=q.device)
    check(lib.ka_sliding_attention(_p(out), _p(q), _p(k_cache), _p(v_cache), _p(block_tables), _p(q_starts),
                                   block_tables.shape[0], *tail(T), 1 if tile and q_starts is None else 0, _stream()),
          "sliding_attention")
    return out


def delta_prep(cv: torch.Tensor, beta_src: torch.Tensor, b_off: int, a_src: torch.Tensor, a_off: int, A_log: torch.Tensor,
               dt_bias: torch.Tensor, H: int, G: int, D: int, channel: bool):
    """The fp32 inputs of the delta rule from the convolved rows cv = [q (G x D) | k (G x D) | ...]:
    qk [T, 2, G, D]: q and k as unit vectors per head, x / sqrt(sum x^2 + 1e-6), q also times D^-1/2;
    beta [T, H] = sigmoid(beta_src[:, b_off : b_off + H]);
    decay = exp(-exp(A_log[h]) * softplus(a + dt_bias)): [T, H] from a = a_src[:, a_off : a_off + H], or, channel,
    [T, H, D] from H * D columns (one decay per head and key channel)."""
    if _ref(cv):
        return ref.delta_prep(cv, beta_src, b_off, a_src, a_off, A_log, dt_bias, H, G, D, channel)
    lib = require_mixers()
    T = cv.shape[0]
    n = H * D if channel else H
    assert cv.is_contiguous() and cv.shape[1] >= 2 * G * D and beta_src.is_contiguous() and a_src.is_contiguous()
    assert beta_src.dtype == cv.dtype == a_src.dtype and b_off + H <= beta_src.shape[1] and a_off + n <= a_src.shape[1]
    assert A_log.dtype == torch.float32 and A_log.numel() == H and dt_bias.dtype == torch.float32 and dt_bias.numel() == n
    qk = torch.empty((T, 2, G, D), dtype=torch.float32, device=cv.device)
    beta = torch.empty((T, H), dtype=torch.float32, device=cv.device)
    decay = torch.empty((T, H, D) if channel else (T, H), dtype=torch.float32, device=cv.device)
    check(lib.ka_delta_prep(_p(qk), _p(beta), _p(decay), _p(cv), cv.shape[1], _p(beta_src), beta_src.shape[1], b_off,
                            _p(a_src), a_src.shape[1], a_off, _p(A_log), _p(dt_bias), T, H, G, D, int(bool(channel)),
                            _f32(cv), _stream()), "delta_prep")
    return qk, beta, decay


DELTA_LANES = 0   # lanes that hold one memory column in delta_scan: 0 = the kernel's choice by head size; 4 / 8 / 16


def delta_scan(qk: torch.Tensor, v_src: torch.Tensor, v_off: int, beta: torch.Tensor, decay: torch.Tensor,
               st_S: torch.Tensor, seq_slots: torch.Tensor, q_starts: Optional[torch.Tensor], positions: torch.Tensor,
               H: int, G: int, D: int, Dv: int) -> torch.Tensor:
    """The gated delta rule over each sequence's rows, from / into the memory of its slot (st_S [slots, H, Dv, D]
    fp32; a sequence whose first row is at position 0 starts from zero, so slots are reused without clearing).
    Per head, with q, k = qk[t, 0 / 1, h // (H / G)], v = v_src[t, v_off + h * Dv ...]:
      S <- decay * S  (decay [T, H]: the whole memory; [T, H, D]: the rows of each key channel)
      u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q.
    q_starts None: row t is sequence t.  -> [T, H * Dv] fp32."""
    if _ref(qk):
        return ref.delta_scan(qk, v_src, v_off, beta, decay, st_S, seq_slots, q_starts, positions, H, G, D, Dv)
    lib = require_mixers()
    T = qk.shape[0]
    nseq = seq_slots.shape[0]
    channel = decay.dim() == 3
    assert qk.dtype == torch.float32 and qk.shape == (T, 2, G, D) and qk.is_contiguous() and H % G == 0
    assert v_src.is_contiguous() and v_off + H * Dv <= v_src.shape[1] and v_src.shape[0] >= T
    assert beta.dtype == decay.dtype == torch.float32 and beta.shape == (T, H) and beta.is_contiguous()
    assert decay.is_contiguous() and decay.shape == ((T, H, D) if channel else (T, H))
    assert st_S.dtype == torch.float32 and st_S.shape[1:] == (H, Dv, D) and st_S.is_contiguous()
    assert seq_slots.dtype == torch.int32 and positions.dtype == torch.int32 and positions.shape[0] >= T
    assert (q_starts is None and nseq <= T) or (q_starts is not None and q_starts.dtype == torch.int32
                                                 and q_starts.shape[0] == nseq + 1)
    out = torch.zeros((T, H * Dv), dtype=torch.float32, device=qk.device)
    check(lib.ka_delta_scan(_p(out), _p(qk), _p(v_src), v_src.shape[1], v_off, _p(beta), _p(decay), _p(st_S),
                            _p(seq_slots), _p(q_starts), nseq, _p(positions), H, G, D, Dv, int(channel), DELTA_LANES,
                            _f32(v_src), _stream()), "delta_scan")
    return out
