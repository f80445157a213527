"""Plain-PyTorch fp32 reference implementations of every engine op.

These define the semantics the HIP kernels (`csrc/*.hip`) must match; the GPU numerics tests
compare kernel output against them, and CPU-only runs (tests, no GPU) execute the engine through
them.  Layouts are documented in `csrc/elementwise.hip` / `csrc/attention.hip`.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch
import torch.nn.functional as F


def linear(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """y = x @ w.T computed in fp32 (the reference for every projection), returned in x's dtype."""
    return torch.nn.functional.linear(x.float(), w.float()).to(x.dtype)


def rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float, residual: Optional[torch.Tensor] = None) -> torch.Tensor:
    if residual is not None:
        r = (x.float() + residual.float()).to(x.dtype)
        residual.copy_(r)
        x = r
    xf = x.float()
    y = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * w.float()
    return y.to(x.dtype)


def rope_cos_sin(max_pos: int, head_dim: int, theta: float, device=None) -> torch.Tensor:
    inv = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float64) / head_dim))
    t = torch.arange(max_pos, dtype=torch.float64)
    f = torch.outer(t, inv)
    return torch.cat([f.cos(), f.sin()], dim=-1).float().to(device)


def rope_kv_write(qkv, positions, cos_sin, slot_mapping, k_cache, v_cache, hq: int, hkv: int, d: int):
    T = qkv.shape[0]
    half = d // 2
    q = qkv[:, : hq * d].view(T, hq, d).float()
    k = qkv[:, hq * d: (hq + hkv) * d].view(T, hkv, d).float()
    v = qkv[:, (hq + hkv) * d:].view(T, hkv, d)
    cs = cos_sin[positions.long()]
    cos, sin = cs[:, None, :half], cs[:, None, half:]

    def rot(x):
        x1, x2 = x[..., :half], x[..., half:]
        return torch.cat([x1 * cos - x2 * sin, x2 * cos + x1 * sin], dim=-1)

    q_out = rot(q).to(qkv.dtype)
    k_rot = rot(k).to(qkv.dtype)
    bs = k_cache.shape[2]
    slots = slot_mapping.long()
    valid = slots >= 0
    if valid.any():
        s = slots[valid]
        blk, off = s // bs, s % bs
        k_cache[blk, :, off, :] = k_rot[valid].to(k_cache.dtype)
        v_cache[blk, :, :, off] = v[valid].to(v_cache.dtype)
    return q_out


def _gather_kv(k_cache, v_cache, table_row, ctx: int):
    bs = k_cache.shape[2]
    nb = (ctx + bs - 1) // bs
    blocks = table_row[:nb].long()
    k = k_cache[blocks]                       # [nb, Hkv, bs, D]
    v = v_cache[blocks].transpose(-1, -2)     # [nb, Hkv, bs, D]
    k = k.permute(1, 0, 2, 3).reshape(k.shape[1], nb * bs, -1)[:, :ctx]
    v = v.permute(1, 0, 2, 3).reshape(v.shape[1], nb * bs, -1)[:, :ctx]
    return k.float(), v.float()               # [Hkv, ctx, D]


def attention_prefill(q, k_cache, v_cache, block_tables, q_starts, ctx_lens, scale: float):
    T, hq, d = q.shape
    hkv = k_cache.shape[1]
    G = hq // hkv
    out = torch.zeros_like(q)
    qs = q_starts.tolist()
    cl = ctx_lens.tolist()
    for s in range(len(cl)):
        q0, q1, ctx = qs[s], qs[s + 1], cl[s]
        qlen = q1 - q0
        if qlen == 0 or ctx == 0:      # ctx 0 = padding row of a bucketed decode batch
            continue
        k, v = _gather_kv(k_cache, v_cache, block_tables[s], ctx)
        k = k.repeat_interleave(G, dim=0)
        v = v.repeat_interleave(G, dim=0)
        qq = q[q0:q1].float().transpose(0, 1)            # [Hq, qlen, D]
        sc = torch.matmul(qq, k.transpose(-1, -2)) * scale  # [Hq, qlen, ctx]
        qpos = torch.arange(ctx - qlen, ctx, device=q.device)
        kpos = torch.arange(ctx, device=q.device)
        sc = sc.masked_fill(kpos[None, None, :] > qpos[None, :, None], float("-inf"))
        p = torch.softmax(sc, dim=-1)
        out[q0:q1] = torch.matmul(p, v).transpose(0, 1).to(q.dtype)
    return out


def attention_decode(q, k_cache, v_cache, block_tables, ctx_lens, scale: float):
    B = q.shape[0]
    starts = torch.arange(B + 1, dtype=torch.int32, device=q.device)
    return attention_prefill(q, k_cache, v_cache, block_tables, starts, ctx_lens, scale)


def silu_mul(gu: torch.Tensor) -> torch.Tensor:
    i = gu.shape[-1] // 2
    g, u = gu[..., :i].float(), gu[..., i:].float()
    return (F.silu(g) * u).to(gu.dtype)


def embedding(ids: torch.Tensor, table: torch.Tensor, vocab_offset: int = 0) -> torch.Tensor:
    local = ids.long() - vocab_offset
    valid = (local >= 0) & (local < table.shape[0])
    out = table[local.clamp(0, table.shape[0] - 1)]
    return out * valid[:, None].to(out.dtype)


def masked_argmax(logits, mask_bits, mask_idx, vocab_offset: int = 0) -> Tuple[torch.Tensor, torch.Tensor]:
    lf = logits.float().clone()
    V = lf.shape[1]
    if mask_bits is not None and mask_idx is not None:
        gid = torch.arange(V, device=logits.device) + vocab_offset
        words = mask_bits[:, gid // 32].long()                      # [M, V]
        allowed = ((words >> (gid % 32)) & 1).bool()
        mi = mask_idx.long().to(logits.device)
        rows = allowed[mi.clamp(min=0)] | (mi < 0)[:, None]
        lf = lf.masked_fill(~rows, float("-inf"))
    idx = torch.argmax(lf, dim=-1)   # documented: first index of the maximum (= kernel tie-break)
    val = lf.gather(1, idx[:, None]).squeeze(1)
    return (idx + vocab_offset).to(torch.int32), val


def moe_topk(router_logits: torch.Tensor, k: int):
    p = torch.softmax(router_logits.float(), dim=-1)
    w, ids = torch.topk(p, k, dim=-1)
    w = w / w.sum(-1, keepdim=True)
    return w, ids.to(torch.int32)


def argmax_combine(vals: torch.Tensor, idxs: torch.Tensor) -> torch.Tensor:
    """[ranks, S] (value, global id) pairs -> [S] int32: the largest value, the lowest id on ties."""
    v = vals.float()
    best = v.max(dim=0, keepdim=True).values
    big = torch.iinfo(torch.int32).max
    cand = torch.where(v == best, idxs.to(torch.int64), torch.full_like(idxs, big, dtype=torch.int64))
    return cand.min(dim=0).values.to(torch.int32)


# ------------------------------------------------------------------------------------------------
# fp32-residual models (models/vivepel.py): the ops of ops/mixers.py on CPU tensors.  Statistics,
# scores and weights in fp32; outputs in the activation dtype.
def group_rmsnorm(x: torch.Tensor, w: torch.Tensor, groups: int, eps: float, out_dtype=None) -> torch.Tensor:
    """Row cut into `groups` equal parts, each divided by sqrt(mean(part^2) + eps); times w."""
    xf = x.float()
    parts = xf.view(xf.shape[0], groups, xf.shape[1] // groups)
    y = (parts / torch.sqrt(parts.pow(2).mean(-1, keepdim=True) + eps)).view_as(xf) * w.float()
    return y.to(out_dtype or x.dtype)


def post_norm_residual(resid, y, w_post, ls, w_next, groups: int, eps: float, out_dtype=None):
    """resid += ls * gnorm(y; w_post) (in place, fp32; ls None: 1); returns gnorm(resid; w_next) in out_dtype (y's by
    default), or None."""
    n = group_rmsnorm(y, w_post, groups, eps, torch.float32)
    resid.add_(ls.float() * n if ls is not None else n)
    return group_rmsnorm(resid, w_next, groups, eps, out_dtype or y.dtype) if w_next is not None else None


def polynorm(z: torch.Tensor, coef: torch.Tensor, eps: float) -> torch.Tensor:
    zf = z.float()
    z2 = zf * zf

    def n(u):
        return u / torch.sqrt(u.pow(2).mean(-1, keepdim=True) + eps)

    c = coef.float()
    return (c[0] * n(zf) + c[1] * n(z2) + c[2] * n(z2 * zf) + c[3]).to(z.dtype)


def headnorm_rope_append(qk, q_w, k_w, inv_freq, positions, slots, k_cache, v_cache, H: int, G: int, D: int,
                         rot: int, eps: float):
    """qk [T, (H + G) * D] -> q [T, H, D] normed + rotated; the normed + rotated keys and the raw keys
    (the values) go to k_cache / v_cache [NB, G, BS, D] at `slots`."""
    T = qk.shape[0]
    x = qk.view(T, H + G, D)
    xf = x.float()
    w = torch.cat([q_w.float().expand(H, D), k_w.float().expand(G, D)])
    y = xf / torch.sqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * w
    half = rot // 2
    if half:
        ang = positions.float()[:, None] * inv_freq.float()[None, :]
        cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
        a, b = y[..., :half], y[..., half:rot]
        y = torch.cat([a * cos - b * sin, b * cos + a * sin, y[..., rot:]], dim=-1)
    y = y.to(qk.dtype)
    bs = k_cache.shape[2]
    s = slots.long()
    ok = s >= 0
    if ok.any():
        k_cache[s[ok] // bs, :, s[ok] % bs, :] = y[ok][:, H:]
        v_cache[s[ok] // bs, :, s[ok] % bs, :] = x[ok][:, H:]
    return y[:, :H].contiguous()


def chunk_attention(q, k_cache, v_cache, block_tables, q_starts, positions, slots, mix, chunk: int, scale: float,
                    cap: float, sink: bool):
    """q [T, H, D] -> [T, H * Dv]; see csrc/attention_chunk.hip for the options."""
    T, H, D = q.shape
    G, bs, Dv = k_cache.shape[1], k_cache.shape[2], v_cache.shape[3]
    rep = H // G
    out = torch.zeros(T, H * Dv, dtype=q.dtype, device=q.device)
    pos_l, slot_l = positions.tolist(), slots.tolist()
    seq_l = list(range(T))
    if q_starts is not None:
        qs = q_starts.tolist()
        seq_l = [0] * T
        for i in range(len(qs) - 1):
            seq_l[qs[i]:qs[i + 1]] = [i] * (qs[i + 1] - qs[i])
    for t in range(T):
        if slot_l[t] < 0:
            continue
        p = pos_l[t]
        start = (p // chunk) * chunk if chunk > 0 else 0
        js = torch.arange(start, p + 1, device=q.device)
        pages = block_tables[seq_l[t]].long()[js // bs]
        k = k_cache[pages, :, js % bs, :].float()             # [n, G, D]
        v = v_cache[pages, :, js % bs, :].float()             # [n, G, Dv]
        k = k.repeat_interleave(rep, dim=1)                   # [n, H, D]
        s = torch.einsum("hd,nhd->hn", q[t].float(), k) * scale
        if cap > 0:
            s = cap * torch.tanh(s / cap)
        m = s.max(dim=1, keepdim=True).values
        if sink:
            m = m.clamp(min=0.0)
        e = torch.exp(s - m)
        w = e / (e.sum(dim=1, keepdim=True) + (torch.exp(-m) if sink else 0.0))
        if mix is not None:
            w = mix.float() @ w
        o = torch.einsum("hn,nhd->hd", w, v.repeat_interleave(rep, dim=1))
        out[t] = o.reshape(-1).to(q.dtype)
    return out


# ------------------------------------------------------------------------------------------------
# Stream (hyper-connection) residuals, mLSTM, latent attention with a window and a sink, grouped expert
# routing (models/kafilorn.py): the ops of ops/mixers.py on CPU tensors, fp32 wherever the kernels are.
def embed_streams(ids: torch.Tensor, table: torch.Tensor, scale: float, streams: int) -> torch.Tensor:
    """table[ids] * scale as fp32, copied into `streams` residual streams: [T, S, W]."""
    x = table[ids.long().clamp(0, table.shape[0] - 1)].float() * scale
    return x[:, None, :].repeat(1, streams, 1).contiguous()


def _layer_norm(u: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    d = u - u.mean(-1, keepdim=True)
    return d / torch.sqrt((d * d).mean(-1, keepdim=True) + eps) * w.float()


def stream_norm(x: torch.Tensor, w_in: torch.Tensor, w: torch.Tensor, eps: float, out_dtype) -> torch.Tensor:
    """LayerNorm (weight, no bias) of u = sum_s w_in[s] x[:, s]."""
    u = torch.einsum("tsw,s->tw", x, w_in.float())
    return _layer_norm(u, w, eps).to(out_dtype)


def stream_update(x, y, mix, out, next_in, next_w, eps: float, out_dtype):
    """x[:, t] <- sum_s mix[s, t] x[:, s] + out[t] * y (in place, all streams from the old ones); returns
    the next sublayer's normed input (stream_norm with next_in / next_w) or None."""
    new = torch.einsum("tsw,sr->trw", x, mix.float()) + out.float()[None, :, None] * y.float()[:, None, :]
    x.copy_(new)
    return stream_norm(x, next_in, next_w, eps, out_dtype) if next_w is not None else None


def relu_sq(z: torch.Tensor) -> torch.Tensor:
    r = torch.relu(z.float())
    return (r * r).to(z.dtype)


def mlstm_gates(h: torch.Tensor, w_if: torch.Tensor, b_if: torch.Tensor, cap: float) -> torch.Tensor:
    """[T, 2H] fp32: the capped log input gates, then the log forget gates logsigmoid(capped)."""
    z = h.float() @ w_if.float().t() + b_if.float()
    if cap > 0:
        z = cap * torch.tanh(z / cap)
    H = z.shape[1] // 2
    return torch.cat([z[:, :H], F.logsigmoid(z[:, H:])], dim=1)


def _seq_of(T: int, q_starts):
    if q_starts is None:
        return [(i, i, i + 1) for i in range(T)]
    qs = q_starts.tolist()
    return [(i, qs[i], qs[i + 1]) for i in range(len(qs) - 1)]


def mlstm_scan(proj, q_off: int, k_off: int, v_off: int, gates, st_S, st_n, st_m, seq_slots, q_starts, positions,
               H: int, D: int, Dv: int, qscale: float) -> torch.Tensor:
    """The recurrence over each sequence's rows of this step, from the state in its slot (zero when the row's
    position is 0) and back into it.  proj rows hold q [H, D], k [H, D], v [H, Dv] at the given column offsets.
    -> (numerators S^T q [T, H * Dv], denominators max(|n . q|, exp(-m)) + 1e-6 [T, H]), fp32."""
    T = proj.shape[0]
    out = torch.zeros((T, H * Dv), dtype=torch.float32, device=proj.device)
    dens = torch.ones((T, H), dtype=torch.float32, device=proj.device)
    slots, pos = seq_slots.tolist(), positions.tolist()
    for i, a, b in _seq_of(T, q_starts):
        sl = slots[i]
        if sl < 0 or b <= a:
            continue
        if pos[a] == 0:
            S, n, m = torch.zeros(H, D, Dv), torch.zeros(H, D), torch.zeros(H)
        else:
            S, n, m = st_S[sl].clone(), st_n[sl].clone(), st_m[sl].clone()
        for t in range(a, b):
            q = proj[t, q_off:q_off + H * D].float().view(H, D) * qscale
            k = proj[t, k_off:k_off + H * D].float().view(H, D)
            v = proj[t, v_off:v_off + H * Dv].float().view(H, Dv)
            ig, fg = gates[t, :H], gates[t, H:]
            m_new = torch.maximum(fg + m, ig)
            fa, ia = torch.exp(fg + m - m_new), torch.exp(ig - m_new)
            S = fa[:, None, None] * S + ia[:, None, None] * (k[:, :, None] * v[:, None, :])
            n = fa[:, None] * n + ia[:, None] * k
            m = m_new
            dens[t] = torch.maximum((n * q).sum(-1).abs(), torch.exp(-m)) + 1e-6
            out[t] = torch.einsum("hdv,hd->hv", S, q).reshape(-1)
        st_S[sl], st_n[sl], st_m[sl] = S, n, m
    return out, dens


def headnorm_gate(o, proj, g_off: int, w, H: int, Dv: int, eps: float, out_dtype, den=None, silu: bool = False) -> torch.Tensor:
    """Each head of o (divided by den [T, H] first, if given) divided by its root mean square, times w, times
    sigmoid(gate columns of proj) (silu: times silu of them)."""
    T = o.shape[0]
    oh = o.view(T, H, Dv)
    if den is not None:
        oh = oh / den[:, :, None]
    y = (oh / torch.sqrt((oh * oh).mean(-1, keepdim=True) + eps)).reshape(T, H * Dv) * w.float()
    g = proj[:, g_off:g_off + H * Dv].float()
    return (y * (F.silu(g) if silu else torch.sigmoid(g))).to(out_dtype)


def _rot(x, positions, inv_freq, dims: int, interleaved: bool = False, mag: float = 1.0):
    """Rotary positions on the first `dims` entries: pairs (i, i + dims/2), or (2i, 2i + 1) when interleaved;
    cos and sin times `mag`."""
    half = dims // 2
    if half == 0:
        return x
    ang = positions.float()[:, None] * inv_freq.float()[None, :]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    c, s = (torch.cos(ang) * mag).view(shape), (torch.sin(ang) * mag).view(shape)
    if interleaved:
        a, b = x[..., 0:dims:2], x[..., 1:dims:2]
        turned = torch.stack([a * c - b * s, b * c + a * s], dim=-1).flatten(-2)
        return torch.cat([turned, x[..., dims:]], dim=-1)
    a, b = x[..., :half], x[..., half:dims]
    return torch.cat([a * c - b * s, b * c + a * s, x[..., dims:]], dim=-1)


def latent_prep(proj, Q: int, R: int, Dr: int, w_q, w_kv, inv_freq, positions, slots, cache, rot_dims: int, eps: float,
                interleaved: bool = False, mag: float = 1.0):
    """proj rows = [query latent Q | key/value latent R | rotated key part Dr] (the last two only with a cache).
    -> the RMS-normed query latent [T, Q] (None when Q is 0); the normed latent and the rotated key part go to
    cache[slot]."""
    cq = None
    if Q:
        cq = proj[:, :Q].float()
        cq = (cq / torch.sqrt((cq * cq).mean(-1, keepdim=True) + eps) * w_q.float()).to(proj.dtype).contiguous()
    if cache is not None:
        c = proj[:, Q:Q + R].float()
        c = c / torch.sqrt((c * c).mean(-1, keepdim=True) + eps) * w_kv.float()
        kr = _rot(proj[:, Q + R:Q + R + Dr].float(), positions[:proj.shape[0]], inv_freq, rot_dims, interleaved, mag)
        row = torch.cat([c, kr], dim=1).to(cache.dtype)
        s = slots[:proj.shape[0]].long()
        ok = s >= 0
        if ok.any():
            bs = cache.shape[1]
            cache[s[ok] // bs, s[ok] % bs] = row[ok]
    return cq


def rope_split_q(q, inv_freq, positions, H: int, D: int, Dr: int, rot_dims: int, interleaved: bool = False,
                 mag: float = 1.0, off: int = 0):
    """The columns off .. off + H * (D + Dr) of q's rows -> (unrotated parts [H, T, D] in q's dtype, rotated parts
    [T, H, Dr] fp32)."""
    T = q.shape[0]
    qh = q[:, off:off + H * (D + Dr)].reshape(T, H, D + Dr)
    qn = qh[:, :, :D].transpose(0, 1).contiguous()
    qr = _rot(qh[:, :, D:].float(), positions[:T], inv_freq, rot_dims, interleaved, mag).contiguous()
    return qn, qr


def head_gate(o, gate_src, g_off: int):
    """o [H, T, Dv] -> [T, H * Dv], head h times sigmoid(gate_src[t, g_off + h]) (gate_src None: the layout only)."""
    H, T, Dv = o.shape
    y = o.transpose(0, 1).float()
    if gate_src is not None:
        y = y * torch.sigmoid(gate_src[:T, g_off:g_off + H].float())[:, :, None]
    return y.reshape(T, H * Dv).to(o.dtype).contiguous()


def window_attention(q_lat, q_rot, cache, block_tables, q_starts, positions, slots, sink, window: int, scale: float):
    """One shared key [R + Dr] per token (multi-query): score = (q_lat . c + q_rot . k_rot) * scale over the
    last `window` positions (0: all), softmax with an optional per-head sink logit in the denominator, values
    = the latent c.  q_lat [H, T, R], q_rot [T, H, Dr] -> [H, T, R] in q_lat's dtype."""
    H, T, R = q_lat.shape
    bs = cache.shape[1]
    out = torch.zeros((H, T, R), dtype=q_lat.dtype, device=q_lat.device)
    pos_l, slot_l = positions.tolist(), slots.tolist()
    for i, a, b in _seq_of(T, q_starts):
        for t in range(a, b):
            if slot_l[t] < 0:
                continue
            p = pos_l[t]
            lo = max(0, p - window + 1) if window > 0 else 0
            js = torch.arange(lo, p + 1)
            rows = cache[block_tables[i].long()[js // bs], js % bs].float()       # [n, R + Dr]
            s = (q_lat[:, t].float() @ rows[:, :R].t() + q_rot[t].float() @ rows[:, R:].t()) * scale
            m = s.max(-1, keepdim=True).values
            if sink is not None:
                m = torch.maximum(m, sink.float()[:, None])
            e = torch.exp(s - m)
            den = e.sum(-1, keepdim=True) + (torch.exp(sink.float()[:, None] - m) if sink is not None else 0.0)
            out[:, t] = ((e / den) @ rows[:, :R]).to(q_lat.dtype)
    return out


def moe_route(h, w_router, correction, top: int, groups: int, keep: int, sigmoid: bool = False, renorm: bool = True):
    """Scores over all experts (softmax of the router logits, or their sigmoids); the choice adds `correction` and is
    limited to the `keep` groups (of `groups` equal groups of neighbours) whose best choice score is largest;
    weights = the chosen experts' scores (without correction), over their sum when renorm.
    -> (ids [T, top] int32, weights [T, top] fp32)."""
    z = h.float() @ w_router.float().t()
    s = torch.sigmoid(z) if sigmoid else torch.softmax(z, dim=-1)
    choice = s + correction.float() if correction is not None else s.clone()
    T, E = s.shape
    if groups > 1:
        best = choice.view(T, groups, E // groups).max(-1).values
        kept = torch.zeros_like(best, dtype=torch.bool).scatter_(1, torch.topk(best, keep, dim=-1).indices, True)
        choice = choice.masked_fill(~kept.repeat_interleave(E // groups, dim=1), float("-inf"))
    ids = torch.topk(choice, top, dim=-1).indices
    w = s.gather(1, ids)
    return ids.to(torch.int32), (w / (w.sum(-1, keepdim=True) + 1e-20) if renorm else w.contiguous())


def silu_mul_scaled(gu: torch.Tensor, row_scale: torch.Tensor) -> torch.Tensor:
    """silu(s g) * (s u) per row with its scale s: the gated unit of an input that was multiplied by s."""
    g, u = gu.float().chunk(2, dim=-1)
    sc = row_scale.float()[:, None]
    return (F.silu(g * sc) * (u * sc)).to(gu.dtype)


def moe_experts(h, w_gu, w_down, ids, w, scale_input: bool = False) -> torch.Tensor:
    """sum_k w[t, k] * down_e(silu(gate_e h) * up_e h), e = ids[t, k]; w_gu [E, 2 ff, W] = gate rows then up
    rows, w_down [E, W, ff].  scale_input: the weight multiplies the expert's input instead,
    sum_k down_e(silu(gate_e (w h)) * up_e (w h)), applied to the two projections' fp32 results.  -> [T, W] fp32."""
    T, W = h.shape
    out = torch.zeros((T, W), dtype=torch.float32, device=h.device)
    for e in torch.unique(ids).tolist():
        tok, slot = torch.nonzero(ids == e, as_tuple=True)
        gu = F.linear(h[tok], w_gu[e])
        if scale_input:
            out.index_add_(0, tok, F.linear(silu_mul_scaled(gu, w[tok, slot]), w_down[e]).float())
        else:
            out.index_add_(0, tok, F.linear(silu_mul(gu), w_down[e]).float() * w[tok, slot][:, None])
    return out


def glu_clamp(gu: torch.Tensor, limit: float, alpha: float) -> torch.Tensor:
    """[T, 2 ff] = gate | up -> g sigmoid(alpha g) (u + 1) with g = min(gate, limit), u = clamp(up, -limit, limit)."""
    g, u = gu.float().chunk(2, dim=-1)
    g = g.clamp(max=limit)
    u = u.clamp(-limit, limit)
    return (g * torch.sigmoid(alpha * g) * (u + 1.0)).to(gu.dtype)


# ------------------------------------------------------------------------------------------------
# Dynamic-Tanh norm, scaled residual sums, short convolutions over state slots, rotary positions with a
# frequency table, sliding-window attention that keeps the first tokens, the gated delta rule
# (models/suvapel.py): the ops of ops/mixers.py on CPU tensors, fp32 wherever the kernels are.
def dyt_norm(x, alpha, w, b, out_dtype):
    """tanh(alpha * x) * w + b (alpha: a one-element tensor)."""
    return (torch.tanh(alpha.float() * x.float()) * w.float() + b.float()).to(out_dtype)


def residual_mix(x, ys, coefs, out_dtype, want_copy: bool, dyt):
    """x += sum_i coefs[i] * ys[i] in place (fp32); -> (x in out_dtype if want_copy, dyt_norm(x, *dyt) if dyt)."""
    acc = None
    for y, c in zip(ys, coefs):
        acc = y.float() * c if acc is None else acc + y.float() * c
    x += acc
    return (x.to(out_dtype) if want_copy else None), (dyt_norm(x, *dyt, out_dtype) if dyt is not None else None)


def rms_residual(x, y, w, mult: float, eps: float, out_dtype, dyt):
    """x += mult * y / sqrt(mean(y^2) + eps) * w in place; -> dyt_norm(x, *dyt) if dyt."""
    yf = y.float()
    x += mult * (yf / torch.sqrt((yf * yf).mean(-1, keepdim=True) + eps) * w.float())
    return dyt_norm(x, *dyt, out_dtype) if dyt is not None else None


def gelu_gate_embed(z, table, ids, col0: int):
    """gelu_tanh(z) * table[ids, col0 : col0 + z.shape[1]]."""
    e = table[ids.long().clamp(0, table.shape[0] - 1), col0:col0 + z.shape[1]].float()
    return (F.gelu(z.float(), approximate="tanh") * e).to(z.dtype)


def silu_mul_bias(proj, off: int, ff: int, bias):
    """silu(proj[:, off : off + ff] + bias[:ff]) * (proj[:, off + ff : off + 2 ff] + bias[ff:])."""
    g = proj[:, off:off + ff].float() + bias[:ff].float()
    u = proj[:, off + ff:off + 2 * ff].float() + bias[ff:].float()
    return (F.silu(g) * u).to(proj.dtype)


def short_conv(proj, off: int, C: int, w, state, seq_slots, q_starts, positions, act: bool):
    """y_t = sum_j w[j] * u_(t - taps + 1 + j) per channel over each sequence's rows (w [taps, C]), u = proj[:, off : off + C];
    inputs before this step come from state[slot] [taps - 1, C] (the sequence's last inputs, newest last), inputs
    before position 0 are zero; the state is then advanced by the step's rows.  act: silu on the result."""
    T = proj.shape[0]
    taps = w.shape[0]
    out = torch.zeros((T, C), dtype=proj.dtype, device=proj.device)
    slots, pos = seq_slots.tolist(), positions.tolist()
    for i, a, b in _seq_of(T, q_starts):
        sl = slots[i] if i < len(slots) else -1
        if sl < 0 or b <= a:
            continue
        u = proj[a:b, off:off + C].float()
        hist = state[sl].float() if taps > 1 else u[:0]
        if pos[a] < taps - 1 and taps > 1:   # what lies before position 0 is zero
            hist = hist.clone()
            hist[:taps - 1 - pos[a]] = 0.0
        full = torch.cat([hist, u])                                   # row r of the step is full[r + taps - 1]
        y = sum(w[j].float() * full[j:j + (b - a)] for j in range(taps))
        out[a:b] = (F.silu(y) if act else y).to(proj.dtype)
        if taps > 1:
            state[sl] = full[-(taps - 1):].to(state.dtype)
    return out


def rope_append(qkv, inv_freq, mag: float, positions, slots, k_cache, v_cache, H: int, G: int, D: int, Dv: int, rot: int,
                q_norm=None, k_norm=None, eps: float = 0.0):
    """Rows [q (H x D) | k (G x D) | v (G x Dv)]: with q_norm / k_norm [D], every q / k head is first divided by its
    root mean square (eps inside the root) and multiplied by that weight; rotary positions (angle = position *
    inv_freq, cos and sin times mag) on the first `rot` entries of every q and k head; -> q [T, H, D]; k and v go to
    the paged cache [NB, G, BS, D] / [NB, G, Dv, BS] at `slots`."""
    T = qkv.shape[0]
    q = qkv[:, :H * D].float().view(T, H, D)
    k = qkv[:, H * D:(H + G) * D].float().view(T, G, D)
    if q_norm is not None:
        q = q / torch.sqrt((q * q).mean(-1, keepdim=True) + eps) * q_norm.float()
    if k_norm is not None:
        k = k / torch.sqrt((k * k).mean(-1, keepdim=True) + eps) * k_norm.float()
    v = qkv[:, (H + G) * D:(H + G) * D + G * Dv].view(T, G, Dv)
    half = rot // 2
    if half:
        ang = positions[:T].float()[:, None] * inv_freq.float()[None, :]
        c, s = (torch.cos(ang) * mag)[:, None, :], (torch.sin(ang) * mag)[:, None, :]

        def turn(x):
            a, b = x[..., :half], x[..., half:rot]
            return torch.cat([a * c - b * s, b * c + a * s, x[..., rot:]], dim=-1)

        q, k = turn(q), turn(k)
    sl = slots[:T].long()
    ok = sl >= 0
    if ok.any():
        bs = k_cache.shape[2]
        k_cache[sl[ok] // bs, :, sl[ok] % bs] = k[ok].to(k_cache.dtype)
        v_cache[sl[ok] // bs, :, :, sl[ok] % bs] = v[ok].to(v_cache.dtype)
    return q.to(qkv.dtype).contiguous()


def sliding_attention(q, k_cache, v_cache, block_tables, q_starts, positions, slots, gate_src, g_off: int, window: int,
                      keep_first: int, scale: float, dist=None):
    """q [T, H, D] -> [T, H * Dv]: softmax attention over the keys j <= p with p - j < window or j < keep_first
    (window 0: all); head h's result times sigmoid(gate_src[t, g_off + h]) (gate_src None: no gate).
    dist [3, H] = (r1, r2, pb): no softmax, a visible key's weight is sigmoid(score - r1 ln(1 + r2 (p - j)) + pb)."""
    T, H, D = q.shape
    G, bs, Dv = k_cache.shape[1], k_cache.shape[2], v_cache.shape[2]
    rep = H // G
    out = torch.zeros(T, H * Dv, dtype=q.dtype, device=q.device)
    pos_l, slot_l = positions.tolist(), slots.tolist()
    for i, a, b in _seq_of(T, q_starts):
        for t in range(a, b):
            if slot_l[t] < 0:
                continue
            p = pos_l[t]
            lo = max(0, p - window + 1) if window > 0 else 0
            js = torch.cat([torch.arange(0, min(keep_first, lo)), torch.arange(lo, p + 1)])
            pages = block_tables[i].long()[js // bs]
            k = k_cache[pages, :, js % bs, :].float().repeat_interleave(rep, dim=1)   # [n, H, D]
            v = v_cache[pages, :, :, js % bs].float().repeat_interleave(rep, dim=1)   # [n, H, Dv]
            sc = torch.einsum("hd,nhd->hn", q[t].float(), k) * scale
            if dist is not None:
                d = (p - js).float()[None, :]
                w = torch.sigmoid(sc - dist[0].float()[:, None] * torch.log1p(dist[1].float()[:, None] * d)
                                  + dist[2].float()[:, None])
            else:
                w = torch.softmax(sc, dim=1)
            o = torch.einsum("hn,nhd->hd", w, v)
            if gate_src is not None:
                o = o * torch.sigmoid(gate_src[t, g_off:g_off + H].float())[:, None]
            out[t] = o.reshape(-1).to(q.dtype)
    return out


def delta_prep(cv, beta_src, b_off: int, a_src, a_off: int, A_log, dt_bias, H: int, G: int, D: int, channel: bool):
    """From the convolved rows cv = [q (G x D) | k (G x D) | ...]: unit q (times D^-1/2) and unit k per head
    (x / sqrt(sum x^2 + 1e-6)) -> qk [T, 2, G, D]; beta = sigmoid(beta_src[:, b_off : b_off + H]) [T, H]; decay =
    exp(-exp(A_log) * softplus(a + dt_bias)) [T, H] (a = a_src[:, a_off : a_off + H]) or, channel, [T, H, D] (a of
    H * D columns).  All fp32."""
    T = cv.shape[0]
    x = cv[:, :2 * G * D].float().view(T, 2, G, D)
    x = x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)
    x[:, 0] *= D ** -0.5
    beta = torch.sigmoid(beta_src[:, b_off:b_off + H].float())
    n = H * D if channel else H
    sp = F.softplus(a_src[:, a_off:a_off + n].float() + dt_bias.float())
    rate = torch.exp(A_log.float())
    decay = torch.exp(-(rate[None, :, None] * sp.view(T, H, D))) if channel else torch.exp(-(rate[None, :] * sp))
    return x.contiguous(), beta.contiguous(), decay.contiguous()


def delta_scan(qk, v_src, v_off: int, beta, decay, st_S, seq_slots, q_starts, positions, H: int, G: int, D: int, Dv: int):
    """The gated delta rule over each sequence's rows, from / into st_S[slot] [H, Dv, D] (zero when the first row's
    position is 0): S <- decay * S (per head or per key channel); u = beta (v - S^T k); S <- S + k u^T; o = S^T q.
    -> [T, H * Dv] fp32."""
    T = qk.shape[0]
    rep = H // G
    out = torch.zeros((T, H * Dv), dtype=torch.float32, device=qk.device)
    slots, pos = seq_slots.tolist(), positions.tolist()
    for i, a, b in _seq_of(T, q_starts):
        sl = slots[i] if i < len(slots) else -1
        if sl < 0 or b <= a:
            continue
        S = torch.zeros(H, Dv, D) if pos[a] == 0 else st_S[sl].clone()
        for t in range(a, b):
            q = qk[t, 0].repeat_interleave(rep, dim=0)      # [H, D]
            k = qk[t, 1].repeat_interleave(rep, dim=0)
            v = v_src[t, v_off:v_off + H * Dv].float().view(H, Dv)
            g = decay[t].view(H, 1, -1)                     # [H, 1, 1 or D]
            S = S * g
            u = beta[t][:, None] * (v - torch.einsum("hvd,hd->hv", S, k))
            S = S + u[:, :, None] * k[:, None, :]
            out[t] = torch.einsum("hvd,hd->hv", S, q).reshape(-1)
        st_S[sl] = S
    return out
