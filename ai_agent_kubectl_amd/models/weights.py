"""Weight creation and loading, tensor/expert-parallel aware.

Fused layouts (row-major `[out, in]`, consumed by `F.linear` / the HIP GEMV):
  wqkv [(Hq + 2 Hkv) * D / t, H]   column-parallel: this rank's q heads, then k heads, then v heads
  wo   [H, Hq * D / t]             row-parallel
  w13  [2 I / t, H]                column-parallel gate | up (each half sharded)
  w2   [H, I / t]                  row-parallel
  MoE: w13 [E_local, 2 I, H], w2 [E_local, H, I], router [E, H] (replicated)
  embed [V, H] replicated; lm_head [V / t, H] vocab-parallel.

Random init (`WEIGHTS=random:<seed>`, the BASELINE configs' "random-init weights") is generated in
*parallel-invariant units* — one seeded draw per attention head, per 1/64 of the MLP width, per
1/64 of the vocab, per expert — so a TP=t shard is bit-identical to the matching slice of the TP=1
weights.  That is what makes the virtual-TP and multi-process TP parity tests exact.

`load_safetensors` maps HF Llama / Mixtral checkpoints (`model.layers.N.self_attn.q_proj.weight`,
...) into the fused, sharded layout.
"""
from __future__ import annotations

import glob
import hashlib
import os
from dataclasses import dataclass
from typing import Dict, List, Optional

import torch

from .config import ModelConfig

STD = 0.02
MLP_UNITS = 64
VOCAB_UNITS = 64


@dataclass
class ParallelInfo:
    tp_rank: int = 0
    tp_size: int = 1
    ep_rank: int = 0
    ep_size: int = 1


def _seed(*parts) -> int:
    h = hashlib.blake2b(repr(parts).encode(), digest_size=8).digest()
    return int.from_bytes(h, "little") & 0x7FFFFFFFFFFFFFFF


def _randn(shape, seed, device, dtype, std=STD):
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    return (torch.randn(shape, generator=g, device=device, dtype=torch.float32) * std).to(dtype)


def _units(total: int, n_units: int, rank: int, size: int) -> List[range]:
    """Split [0,total) into n_units equal units (requires divisibility) and return this rank's unit ranges."""
    assert total % n_units == 0 and n_units % size == 0, (total, n_units, size)
    per = n_units // size
    u = total // n_units
    return [range((rank * per + i) * u, (rank * per + i + 1) * u) for i in range(per)]


def _mlp_units(inter: int) -> int:
    for n in (MLP_UNITS, 32, 16, 8, 4, 2, 1):
        if inter % n == 0:
            return n
    return 1


def _vocab_units(vocab: int) -> int:
    for n in (VOCAB_UNITS, 32, 16, 8, 4, 2, 1):
        if vocab % n == 0:
            return n
    return 1


def validate_parallel(cfg: ModelConfig, par: ParallelInfo) -> None:
    t = par.tp_size
    if cfg.num_heads % t or cfg.num_kv_heads % t:
        raise ValueError(f"TP={t} must divide heads {cfg.num_heads}/{cfg.num_kv_heads}")
    if cfg.is_moe:
        if cfg.num_experts % par.ep_size:
            raise ValueError(f"EP={par.ep_size} must divide experts {cfg.num_experts}")
    elif _mlp_units(cfg.intermediate) % t:
        raise ValueError(f"TP={t} must divide MLP units")
    if _vocab_units(cfg.vocab_size) % t:
        raise ValueError(f"TP={t} must divide the vocab units ({cfg.vocab_size})")


def random_weights(cfg: ModelConfig, par: ParallelInfo, seed: int = 0, device="cpu",
                   dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    validate_parallel(cfg, par)
    H, D = cfg.hidden, cfg.head_dim
    t, r = par.tp_size, par.tp_rank
    hq, hkv = cfg.num_heads // t, cfg.num_kv_heads // t
    W: Dict[str, torch.Tensor] = {}
    W["embed"] = torch.cat([_randn((len(u), H), _seed(seed, "embed", u.start), device, dtype)
                            for u in _units(cfg.vocab_size, _vocab_units(cfg.vocab_size), 0, 1)])
    W["lm_head"] = torch.cat([_randn((len(u), H), _seed(seed, "lm_head", u.start), device, dtype)
                              for u in _units(cfg.vocab_size, _vocab_units(cfg.vocab_size), r, t)])
    W["norm"] = torch.ones(H, device=device, dtype=dtype)
    for L in range(cfg.num_layers):
        p = f"layers.{L}."
        q = [_randn((D, H), _seed(seed, L, "q", r * hq + i), device, dtype) for i in range(hq)]
        k = [_randn((D, H), _seed(seed, L, "k", r * hkv + i), device, dtype) for i in range(hkv)]
        v = [_randn((D, H), _seed(seed, L, "v", r * hkv + i), device, dtype) for i in range(hkv)]
        W[p + "wqkv"] = torch.cat(q + k + v)
        W[p + "wo"] = torch.cat([_randn((H, D), _seed(seed, L, "o", r * hq + i), device, dtype)
                                 for i in range(hq)], dim=1)
        W[p + "ln1"] = torch.ones(H, device=device, dtype=dtype)
        W[p + "ln2"] = torch.ones(H, device=device, dtype=dtype)
        if cfg.is_moe:
            E = cfg.num_experts
            W[p + "router"] = _randn((E, H), _seed(seed, L, "router"), device, dtype)
            el = E // par.ep_size
            w13, w2 = [], []
            for i in range(el):
                e = par.ep_rank * el + i
                g = _randn((cfg.intermediate, H), _seed(seed, L, "e_gate", e), device, dtype)
                u_ = _randn((cfg.intermediate, H), _seed(seed, L, "e_up", e), device, dtype)
                w13.append(torch.cat([g, u_]))
                w2.append(_randn((H, cfg.intermediate), _seed(seed, L, "e_down", e), device, dtype))
            W[p + "w13"] = torch.stack(w13)
            W[p + "w2"] = torch.stack(w2)
        else:
            units = _units(cfg.intermediate, _mlp_units(cfg.intermediate), r, t)
            gate = [_randn((len(u), H), _seed(seed, L, "gate", u.start), device, dtype) for u in units]
            up = [_randn((len(u), H), _seed(seed, L, "up", u.start), device, dtype) for u in units]
            W[p + "w13"] = torch.cat(gate + up)
            W[p + "w2"] = torch.cat([_randn((H, len(u)), _seed(seed, L, "down", u.start), device, dtype)
                                     for u in units], dim=1)
    return W


# ------------------------------------------------------------------------------------------------
def load_safetensors(path: str, cfg: ModelConfig, par: ParallelInfo, device="cpu",
                     dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """Load an HF-format Llama / Mixtral checkpoint (one file or a directory of shards)."""
    from safetensors import safe_open

    validate_parallel(cfg, par)
    files = [path] if os.path.isfile(path) else sorted(glob.glob(os.path.join(path, "*.safetensors")))
    if not files:
        raise FileNotFoundError(f"no .safetensors under {path}")
    handles = [safe_open(f, framework="pt", device="cpu") for f in files]
    index = {}
    for hnd in handles:
        for k in hnd.keys():
            index[k] = hnd

    def get(name) -> torch.Tensor:
        return index[name].get_tensor(name)

    t, r = par.tp_size, par.tp_rank
    D, H = cfg.head_dim, cfg.hidden
    hq, hkv = cfg.num_heads // t, cfg.num_kv_heads // t

    def rows(x, start, n):
        return x[start:start + n]

    W: Dict[str, torch.Tensor] = {}
    W["embed"] = get("model.embed_tokens.weight")
    lm = get("lm_head.weight") if "lm_head.weight" in index else W["embed"]
    vs = cfg.vocab_size // t
    W["lm_head"] = rows(lm, r * vs, vs)
    W["norm"] = get("model.norm.weight")
    for L in range(cfg.num_layers):
        p, hp = f"layers.{L}.", f"model.layers.{L}."
        q = rows(get(hp + "self_attn.q_proj.weight"), r * hq * D, hq * D)
        k = rows(get(hp + "self_attn.k_proj.weight"), r * hkv * D, hkv * D)
        v = rows(get(hp + "self_attn.v_proj.weight"), r * hkv * D, hkv * D)
        W[p + "wqkv"] = torch.cat([q, k, v])
        W[p + "wo"] = get(hp + "self_attn.o_proj.weight")[:, r * hq * D:(r + 1) * hq * D]
        W[p + "ln1"] = get(hp + "input_layernorm.weight")
        W[p + "ln2"] = get(hp + "post_attention_layernorm.weight")
        if cfg.is_moe:
            W[p + "router"] = get(hp + "block_sparse_moe.gate.weight")
            el = cfg.num_experts // par.ep_size
            w13, w2 = [], []
            for i in range(el):
                e = par.ep_rank * el + i
                ep = hp + f"block_sparse_moe.experts.{e}."
                w13.append(torch.cat([get(ep + "w1.weight"), get(ep + "w3.weight")]))
                w2.append(get(ep + "w2.weight"))
            W[p + "w13"] = torch.stack(w13)
            W[p + "w2"] = torch.stack(w2)
        else:
            i_l = cfg.intermediate // t
            g = rows(get(hp + "mlp.gate_proj.weight"), r * i_l, i_l)
            u = rows(get(hp + "mlp.up_proj.weight"), r * i_l, i_l)
            W[p + "w13"] = torch.cat([g, u])
            W[p + "w2"] = get(hp + "mlp.down_proj.weight")[:, r * i_l:(r + 1) * i_l]
    return {k: v.to(device=device, dtype=dtype).contiguous() for k, v in W.items()}


# ------------------------------------------------------------------------------------------------
# Vivepel.  Engine layout per layer `layers.<i>.`: wqk [(H + G) * D, W] with bias bqk (the q rows, then
# the k rows: one GEMM), wo [W, H * Dv], w_up [ff, W], w_down [W, ff] in the activation dtype; the
# norm weights (norm1, norm1b, norm2, norm2b, q_norm, k_norm), the layer scales (ls1, ls2), the head
# mixing matrix (talk), the PolyNorm coefficients (act) and the rotary frequencies (inv_freq) in fp32,
# because the ops that read them compute in fp32.
_VIVEPEL_F32 = ("norm1", "norm1b", "norm2", "norm2b", "ls1", "ls2", "q_norm", "k_norm", "talk", "act", "inv_freq")


def _vivepel_pack(cfg, get, device, dtype) -> Dict[str, torch.Tensor]:
    """get(checkpoint name) -> tensor; returns the engine layout on `device`."""
    W: Dict[str, torch.Tensor] = {"embed": get("embed"), "lm_head": get("head"), "norm": get("final.norm").float()}
    for i, L in enumerate(cfg.layers):
        p, c, m = f"layers.{i}.", f"l{i}.", L.mixer
        W[p + "wqk"] = torch.cat([get(c + "mix.q"), get(c + "mix.k")])
        W[p + "bqk"] = torch.cat([get(c + "mix.q.b"), get(c + "mix.k.b")])
        W[p + "wo"] = get(c + "mix.o")
        W[p + "q_norm"], W[p + "k_norm"] = get(c + "mix.q.norm"), get(c + "mix.k.norm")
        W[p + "talk"] = get(c + "mix.talk")
        for k in ("norm1", "norm1b", "ls1"):
            W[p + k] = get(c + k)
        half = m.rot_dims // 2
        # base^(-2i / dims) in float64, rounded once to fp32; the angle is position * inv_freq in fp32
        W[p + "inv_freq"] = (float(m.rot_base) ** (-2.0 * torch.arange(half, dtype=torch.float64) / max(m.rot_dims, 1)))
        if L.ff:
            W[p + "w_up"], W[p + "w_down"], W[p + "act"] = get(c + "mlp.up"), get(c + "mlp.down"), get(c + "mlp.act")
            for k in ("norm2", "norm2b", "ls2"):
                W[p + k] = get(c + k)
    out = {}
    for k, v in W.items():
        f32 = k == "norm" or k.rsplit(".", 1)[-1] in _VIVEPEL_F32
        out[k] = v.to(device=device, dtype=torch.float32 if f32 else dtype).contiguous()
    return out


def vivepel_check_shapes(cfg, W: Dict[str, torch.Tensor]) -> None:
    """Every tensor of the engine layout has the shape the configuration implies."""
    h, V = cfg.hidden, cfg.vocab_size
    want = {"embed": (V, h), "lm_head": (V, h), "norm": (h,)}
    for i, L in enumerate(cfg.layers):
        p, m = f"layers.{i}.", L.mixer
        n = (m.heads + m.kv_heads) * m.dim
        want.update({p + "wqk": (n, h), p + "bqk": (n,), p + "wo": (h, m.heads * m.vdim), p + "q_norm": (m.dim,),
                     p + "k_norm": (m.dim,), p + "talk": (m.heads, m.heads), p + "norm1": (h,), p + "norm1b": (h,),
                     p + "ls1": (h,), p + "inv_freq": (m.rot_dims // 2,)})
        if L.ff:
            want.update({p + "w_up": (L.ff, h), p + "w_down": (h, L.ff), p + "act": (4,), p + "norm2": (h,),
                         p + "norm2b": (h,), p + "ls2": (h,)})
    for k, shp in want.items():
        if k not in W or tuple(W[k].shape) != shp:
            raise ValueError(f"tensor {k}: expected shape {shp}, found {tuple(W[k].shape) if k in W else None}")


def vivepel_checkpoint_tensors(cfg, seed: int = 0, dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """Random tensors under the checkpoint's own names (what a Vivepel model.safetensors holds)."""
    g = torch.Generator().manual_seed(_seed(seed, "vivepel") & 0x7FFFFFFF)
    h, V = cfg.hidden, cfg.vocab_size

    def mat(o, i, std=None):
        return (torch.randn(o, i, generator=g) * (std if std is not None else i ** -0.5)).to(dtype)

    def vec(n, lo=0.75, hi=1.25):
        return (lo + (hi - lo) * torch.rand(n, generator=g)).to(dtype)

    T = {"embed": mat(V, h, 1.0), "head": mat(V, h), "final.norm": vec(h)}
    for i, L in enumerate(cfg.layers):
        c, m = f"l{i}.", L.mixer
        T[c + "mix.q"], T[c + "mix.q.b"] = mat(m.heads * m.dim, h), (torch.randn(m.heads * m.dim, generator=g) * 0.1).to(dtype)
        T[c + "mix.k"], T[c + "mix.k.b"] = mat(m.kv_heads * m.dim, h), (torch.randn(m.kv_heads * m.dim, generator=g) * 0.1).to(dtype)
        T[c + "mix.q.norm"], T[c + "mix.k.norm"] = vec(m.dim), vec(m.dim)
        T[c + "mix.talk"] = (torch.eye(m.heads) * 0.8 + torch.randn(m.heads, m.heads, generator=g) * (0.2 / m.heads ** 0.5)).to(dtype)
        T[c + "mix.o"] = mat(h, m.heads * m.vdim)
        for k in ("norm1", "norm1b"):
            T[c + k] = vec(h)
        T[c + "ls1"] = vec(h, 0.2, 0.6)
        if L.ff:
            T[c + "mlp.up"], T[c + "mlp.down"] = mat(L.ff, h), mat(h, L.ff)
            T[c + "mlp.act"] = torch.tensor([0.6, 0.3, 0.15, 0.02]).to(dtype)
            for k in ("norm2", "norm2b"):
                T[c + k] = vec(h)
            T[c + "ls2"] = vec(h, 0.2, 0.6)
    return T


def vivepel_random_weights(cfg, seed: int = 0, device="cpu", dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """Random-init Vivepel weights: drawn in bf16 (as a checkpoint stores them), packed for `dtype`."""
    T = vivepel_checkpoint_tensors(cfg, seed)
    W = _vivepel_pack(cfg, T.__getitem__, device, dtype)
    vivepel_check_shapes(cfg, W)
    return W


def load_vivepel_safetensors(path: str, cfg, device="cpu", dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """A Vivepel checkpoint (a file, or a folder holding model.safetensors / *.safetensors)."""
    from safetensors import safe_open

    files = [path] if os.path.isfile(path) else sorted(glob.glob(os.path.join(path, "*.safetensors")))
    if not files:
        raise FileNotFoundError(f"no .safetensors under {path}")
    index = {}
    for f in files:
        hnd = safe_open(f, framework="pt", device="cpu")
        for k in hnd.keys():
            index[k] = hnd

    def get(name):
        if name not in index:
            raise KeyError(f"{path}: tensor {name!r} is missing")
        return index[name].get_tensor(name)

    W = _vivepel_pack(cfg, get, device, dtype)
    vivepel_check_shapes(cfg, W)
    return W


# ------------------------------------------------------------------------------------------------
# Kafilorn.  Engine layout per layer `layers.<i>.` (activation dtype unless marked fp32):
#   norm1, norm2, hc{1,2}_in [S], hc{1,2}_out [S], hc{1,2}_mix [S, S]                         fp32
#   mLSTM:  w_proj [q; k; v; g rows, W] (one GEMM), w_if [2H, W] + b_if [2H] fp32 (input gates, then forget
#           gates; w_if_lp: the checkpoint's bf16 values of w_if, bf16 engine only), hnorm [H * Dv] fp32, wo [W, H * Dv]
#   latent attention:  w_dn [dq rows; dkv rows, W] (one GEMM; dq alone when the layer borrows another layer's
#           cache), q_norm [Q] / kv_norm [R] / sink [H] / inv_freq fp32, w_uq [H * (D + Dr), Q],
#           w_uk [H, D, R], w_uv [H, Dv, R], wo [W, H * Dv]
#   dense feed-forward:  w_up [ff, W], w_down [W, ff]
#   experts:  w_router [E, W] + correction [E] fp32, w_gu [E, 2 ff, W] (gate rows, then up rows),
#           w_dn_e [E, W, ff], shared expert ws_gu [2 sff, W], ws_down [W, sff]
# A model without streams is stored with S = 1 and unit stream weights (the plain residual sum).
_KAFILORN_F32 = ("norm1", "norm2", "hc1_in", "hc1_out", "hc1_mix", "hc2_in", "hc2_out", "hc2_mix", "w_if", "b_if", "hnorm",
                 "q_norm", "kv_norm", "sink", "inv_freq", "w_router", "correction")


def _kafilorn_pack(cfg, get, device, dtype) -> Dict[str, torch.Tensor]:
    S = max(cfg.streams, 1)

    def opt(name, n):   # a tensor the checkpoint may leave out: zeros (no correction, a sink of weight exp(0))
        try:
            return get(name)
        except KeyError:
            return torch.zeros(n)

    W: Dict[str, torch.Tensor] = {"embed": get("embed"), "lm_head": get("head"), "norm": get("final.norm").float(),
                                  "ones": torch.ones(S)}
    for i, L in enumerate(cfg.layers):
        p, c, m, f = f"layers.{i}.", f"l{i}.", L.mixer, L.mlp
        for q in ("1", "2") if f is not None else ("1",):
            W[p + "norm" + q] = get(c + "norm" + q)
            for k in ("in", "out", "mix"):
                W[p + f"hc{q}_{k}"] = get(c + f"hc{q}.{k}") if cfg.streams else torch.ones((1, 1) if k == "mix" else (1,))
        if m.kind == "mlstm":
            W[p + "w_proj"] = torch.cat([get(c + "mix.q"), get(c + "mix.k"), get(c + "mix.v"), get(c + "mix.g")])
            W[p + "w_if"] = torch.cat([get(c + "mix.i"), get(c + "mix.f")])
            W[p + "b_if"] = torch.cat([get(c + "mix.i.b"), get(c + "mix.f.b")])
            if dtype == torch.bfloat16 and W[p + "w_if"].dtype == torch.bfloat16:
                W[p + "w_if_lp"] = W[p + "w_if"]    # the stored bf16 values, for the matrix cores (w_if becomes fp32 below)
            W[p + "hnorm"], W[p + "wo"] = get(c + "mix.norm"), get(c + "mix.o")
        else:
            own = m.kv_from < 0
            W[p + "w_dn"] = torch.cat([get(c + "mix.dq"), get(c + "mix.dkv")]) if own else get(c + "mix.dq")
            W[p + "q_norm"] = get(c + "mix.dq.norm")
            if own:
                W[p + "kv_norm"] = get(c + "mix.dkv.norm")
            W[p + "w_uq"] = get(c + "mix.uq")
            W[p + "w_uk"] = get(c + "mix.uk").view(m.heads, m.dim, m.kv_rank)
            W[p + "w_uv"] = get(c + "mix.uv").view(m.heads, m.vdim, m.kv_rank)
            W[p + "sink"], W[p + "wo"] = get(c + "mix.sink"), get(c + "mix.o")
            half = m.rot_dims // 2
            # base^(-2i / dims) in float64, rounded once to fp32; the angle is position * inv_freq in fp32
            W[p + "inv_freq"] = float(m.rot_base) ** (-2.0 * torch.arange(half, dtype=torch.float64) / max(m.rot_dims, 1))
        if f is None:
            continue
        if f.kind == "dense":
            W[p + "w_up"], W[p + "w_down"] = get(c + "mlp.up"), get(c + "mlp.down")
        else:
            W[p + "w_router"], W[p + "correction"] = get(c + "mlp.router"), opt(c + "mlp.correction", f.experts)
            W[p + "w_gu"] = torch.stack([torch.cat([get(c + f"mlp.e{e}.gate"), get(c + f"mlp.e{e}.up")]) for e in range(f.experts)])
            W[p + "w_dn_e"] = torch.stack([get(c + f"mlp.e{e}.down") for e in range(f.experts)])
            if f.shared_ff:
                W[p + "ws_gu"] = torch.cat([get(c + "mlp.shared.gate"), get(c + "mlp.shared.up")])
                W[p + "ws_down"] = get(c + "mlp.shared.down")
    out = {}
    for k, v in W.items():
        f32 = k in ("norm", "ones") or k.rsplit(".", 1)[-1] in _KAFILORN_F32
        out[k] = v.to(device=device, dtype=torch.float32 if f32 else dtype).contiguous()
    return out


def kafilorn_check_shapes(cfg, W: Dict[str, torch.Tensor]) -> None:
    """Every tensor of the engine layout has the shape the configuration implies."""
    h, V, S = cfg.hidden, cfg.vocab_size, max(cfg.streams, 1)
    want = {"embed": (V, h), "lm_head": (V, h), "norm": (h,)}
    for i, L in enumerate(cfg.layers):
        p, m, f = f"layers.{i}.", L.mixer, L.mlp
        for q in ("1", "2") if f is not None else ("1",):
            want.update({p + "norm" + q: (h,), p + f"hc{q}_in": (S,), p + f"hc{q}_out": (S,), p + f"hc{q}_mix": (S, S)})
        if m.kind == "mlstm":
            want.update({p + "w_proj": (2 * m.heads * (m.dim + m.vdim), h), p + "w_if": (2 * m.heads, h),
                         p + "b_if": (2 * m.heads,), p + "hnorm": (m.heads * m.vdim,), p + "wo": (h, m.heads * m.vdim)})
        else:
            own = m.kv_from < 0
            want.update({p + "w_dn": (m.q_rank + (m.kv_rank + m.rot_dim if own else 0), h), p + "q_norm": (m.q_rank,),
                         p + "w_uq": (m.heads * (m.dim + m.rot_dim), m.q_rank), p + "w_uk": (m.heads, m.dim, m.kv_rank),
                         p + "w_uv": (m.heads, m.vdim, m.kv_rank), p + "sink": (m.heads,), p + "wo": (h, m.heads * m.vdim),
                         p + "inv_freq": (m.rot_dims // 2,)})
            if own:
                want[p + "kv_norm"] = (m.kv_rank,)
        if f is not None and f.kind == "dense":
            want.update({p + "w_up": (f.ff, h), p + "w_down": (h, f.ff)})
        elif f is not None:
            want.update({p + "w_router": (f.experts, h), p + "correction": (f.experts,), p + "w_gu": (f.experts, 2 * f.ff, h),
                         p + "w_dn_e": (f.experts, h, f.ff)})
            if f.shared_ff:
                want.update({p + "ws_gu": (2 * f.shared_ff, h), p + "ws_down": (h, f.shared_ff)})
    for k, shp in want.items():
        if k not in W or tuple(W[k].shape) != shp:
            raise ValueError(f"tensor {k}: expected shape {shp}, found {tuple(W[k].shape) if k in W else None}")


def kafilorn_checkpoint_tensors(cfg, seed: int = 0, dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """Random tensors under the checkpoint's own names (what a Kafilorn model.safetensors holds)."""
    g = torch.Generator().manual_seed(_seed(seed, "kafilorn") & 0x7FFFFFFF)
    h, V, S = cfg.hidden, cfg.vocab_size, cfg.streams

    def mat(o, i, std=None):
        return (torch.randn(o, i, generator=g) * (std if std is not None else i ** -0.5)).to(dtype)

    def vec(n, lo=0.75, hi=1.25):
        return (lo + (hi - lo) * torch.rand(n, generator=g)).to(dtype)

    T = {"embed": mat(V, h, 1.0), "head": mat(V, h), "final.norm": vec(h)}
    for i, L in enumerate(cfg.layers):
        c, m, f = f"l{i}.", L.mixer, L.mlp
        for q in ("1", "2") if f is not None else ("1",):
            T[c + "norm" + q] = vec(h)
            if S:
                T[c + f"hc{q}.in"] = vec(S, 0.5 / S, 1.5 / S)
                T[c + f"hc{q}.out"] = vec(S, 0.5, 1.0)
                T[c + f"hc{q}.mix"] = (torch.eye(S) * 0.8 + torch.rand(S, S, generator=g) * (0.2 / S)).to(dtype)
        if m.kind == "mlstm":
            for k, n in (("q", m.dim), ("k", m.dim), ("v", m.vdim), ("g", m.vdim)):
                T[c + "mix." + k] = mat(m.heads * n, h)
            T[c + "mix.i"], T[c + "mix.f"] = mat(m.heads, h), mat(m.heads, h)
            T[c + "mix.i.b"] = (torch.randn(m.heads, generator=g) * 0.5).to(dtype)
            T[c + "mix.f.b"] = (3.0 + torch.randn(m.heads, generator=g)).to(dtype)
            T[c + "mix.norm"], T[c + "mix.o"] = vec(m.heads * m.vdim), mat(h, m.heads * m.vdim)
        else:
            T[c + "mix.dq"], T[c + "mix.dq.norm"] = mat(m.q_rank, h), vec(m.q_rank)
            T[c + "mix.uq"] = mat(m.heads * (m.dim + m.rot_dim), m.q_rank)
            if m.kv_from < 0:
                T[c + "mix.dkv"], T[c + "mix.dkv.norm"] = mat(m.kv_rank + m.rot_dim, h), vec(m.kv_rank)
            T[c + "mix.uk"], T[c + "mix.uv"] = mat(m.heads * m.dim, m.kv_rank), mat(m.heads * m.vdim, m.kv_rank)
            T[c + "mix.sink"] = torch.randn(m.heads, generator=g).to(dtype)
            T[c + "mix.o"] = mat(h, m.heads * m.vdim)
        if f is not None and f.kind == "dense":
            T[c + "mlp.up"], T[c + "mlp.down"] = mat(f.ff, h), mat(h, f.ff)
        elif f is not None:
            T[c + "mlp.router"] = mat(f.experts, h, 2.0 * h ** -0.5)
            T[c + "mlp.correction"] = (torch.randn(f.experts, generator=g) * (0.5 / f.experts)).to(dtype)
            for e in list(range(f.experts)) + (["shared"] if f.shared_ff else []):
                n, ff = (f"mlp.e{e}.", f.ff) if e != "shared" else ("mlp.shared.", f.shared_ff)
                T[c + n + "gate"], T[c + n + "up"], T[c + n + "down"] = mat(ff, h), mat(ff, h), mat(h, ff)
    return T


def kafilorn_random_weights(cfg, seed: int = 0, device="cpu", dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """Random-init Kafilorn weights: drawn in bf16 (as a checkpoint stores them), packed for `dtype`."""
    T = kafilorn_checkpoint_tensors(cfg, seed)
    W = _kafilorn_pack(cfg, T.__getitem__, device, dtype)
    kafilorn_check_shapes(cfg, W)
    return W


def _safetensors_getter(path: str):
    from safetensors import safe_open

    files = [path] if os.path.isfile(path) else sorted(glob.glob(os.path.join(path, "*.safetensors")))
    if not files:
        raise FileNotFoundError(f"no .safetensors under {path}")
    index = {}
    for f in files:
        hnd = safe_open(f, framework="pt", device="cpu")
        for k in hnd.keys():
            index[k] = hnd

    def get(name):
        if name not in index:
            raise KeyError(f"{path}: tensor {name!r} is missing")
        return index[name].get_tensor(name)

    return get


def load_kafilorn_safetensors(path: str, cfg, device="cpu", dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """A Kafilorn checkpoint (a file, or a folder holding model.safetensors / *.safetensors)."""
    W = _kafilorn_pack(cfg, _safetensors_getter(path), device, dtype)
    kafilorn_check_shapes(cfg, W)
    return W


# ------------------------------------------------------------------------------------------------
# Suvapel.  Engine layout per layer `layers.<i>.` (activation dtype unless marked fp32):
#   norm_w, norm_b [W], norm_alpha [1]                                                         fp32
#   w_in [P, W]: every projection that reads the layer's normed row, stacked for one GEMM, each segment padded
#           with zero rows to a multiple of 8 columns (`suvapel_columns`): attention q | k | v | head gates,
#           delta q | k | v | beta | decay (per head, or the low-rank pair's first half) | output gate (full, or the
#           low-rank pair's first half), feed-forward gate | up
#   att_conv [taps, q + k + v channels], conv [taps, q + k + v channels]  (tap-major)           fp32
#   inv_freq [rot dims / 2] fp32 (YaRN-scaled, float64 rounded once), att_wo [W, H * Dv]
#   A_log [H], dt_bias [H] or [H * D], hnorm [H * Dv] (the shared [Dv] weight repeated per head)  fp32
#   w_a2 [H * D, R], w_g2 [H * Dv, R] (channel decay only), wo [W, H * Dv]
#   b_gu [2 ff] fp32, w_down [W, ff], b_down [W]
#   side_gate [dim, W], side_proj [W, dim], side_norm [W] fp32
# Global: embed, lm_head, side_embed [V, L * dim], norm_w / norm_b / norm_alpha (the final norm).
_SUVAPEL_F32 = ("norm_w", "norm_b", "norm_alpha", "att_conv", "conv", "inv_freq", "A_log", "dt_bias", "hnorm", "b_gu",
                "side_norm")


def _pad8(n: int) -> int:
    return (n + 7) // 8 * 8


def suvapel_columns(L, rank_a: int = 0, rank_g: int = 0) -> Dict[str, int]:
    """Column offsets of a layer's fused input projection (segment name -> first column; "total": the row length).
    rank_a / rank_g: inner sizes of the channel-decay and output-gate pairs (ignored for a per-head decay)."""
    col, o = {}, 0

    def seg(name, n):
        nonlocal o
        col[name] = o
        o += _pad8(n)

    a, m = L.attention, L.delta
    if a is not None:
        seg("att_q", a.heads * a.dim + a.kv_heads * (a.dim + a.vdim))   # q | k | v contiguous: one convolution
        seg("att_g", a.heads)
    seg("q", m.conv_channels())                                         # q | k | v contiguous
    seg("beta", m.heads)
    seg("a", rank_a if m.channel_decay else m.heads)
    seg("g", rank_g if m.channel_decay else m.heads * m.vdim)
    if L.ff:
        seg("ff", 2 * L.ff)                                             # gate | up contiguous
    # the vendor GEMM runs whole 256-column tiles fastest: a wide row block is padded with zero rows to whole tiles
    col["total"] = (o + 1023) // 1024 * 1024 if o >= 8192 else ((o + 255) // 256 * 256 if o >= 2048 else o)
    return col


def _suvapel_pack(cfg, get, device, dtype) -> Dict[str, torch.Tensor]:
    h = cfg.hidden
    W: Dict[str, torch.Tensor] = {"embed": get("embed"), "lm_head": get("head"), "norm_w": get("final.norm"),
                                  "norm_b": get("final.norm.b"), "norm_alpha": get("final.norm.alpha").reshape(1)}
    if cfg.side_dim:
        W["side_embed"] = get("side.embed")
    for i, L in enumerate(cfg.layers):
        p, c, m, a = f"layers.{i}.", f"l{i}.", L.delta, L.attention
        W[p + "norm_w"], W[p + "norm_b"] = get(c + "norm1"), get(c + "norm1.b")
        W[p + "norm_alpha"] = get(c + "norm1.alpha").reshape(1)
        r = c + ("mix.right." if a is not None else "mix.")
        rank_a = get(r + "a1").shape[0] if m.channel_decay else 0
        rank_g = get(r + "g1").shape[0] if m.channel_decay else 0
        col = suvapel_columns(L, rank_a, rank_g)
        w_in = torch.zeros((col["total"], h), dtype=get(r + "q").dtype)

        def put(name, *tensors):
            t = torch.cat(tensors)
            w_in[col[name]:col[name] + t.shape[0]] = t

        if a is not None:
            l = c + "mix.left."
            put("att_q", get(l + "q"), get(l + "k"), get(l + "v"))
            put("att_g", get(l + "g"))
            W[p + "att_conv"] = torch.cat([get(l + "q.conv"), get(l + "k.conv"), get(l + "v.conv")]).t()
            W[p + "att_wo"] = get(l + "o")
            W[p + "inv_freq"] = torch.tensor(a.rot.frequencies()[0], dtype=torch.float64)
        put("q", get(r + "q"), get(r + "k"), get(r + "v"))
        put("beta", get(r + "b"))
        put("a", get(r + "a1") if m.channel_decay else get(r + "a"))
        put("g", get(r + "g1") if m.channel_decay else get(r + "g"))
        W[p + "conv"] = torch.cat([get(r + "q.conv"), get(r + "k.conv"), get(r + "v.conv")]).t()
        W[p + "A_log"], W[p + "dt_bias"] = get(r + "A_log"), get(r + "dt_bias")
        W[p + "hnorm"] = get(r + "norm").repeat(m.heads)
        if m.channel_decay:
            W[p + "w_a2"], W[p + "w_g2"] = get(r + "a2"), get(r + "g2")
        W[p + "wo"] = get(r + "o")
        if L.ff:
            put("ff", get(c + "mlp.gate"), get(c + "mlp.up"))
            W[p + "b_gu"] = torch.cat([get(c + "mlp.gate.b"), get(c + "mlp.up.b")])
            W[p + "w_down"], W[p + "b_down"] = get(c + "mlp.down"), get(c + "mlp.down.b")
        if cfg.side_dim:
            W[p + "side_gate"], W[p + "side_proj"], W[p + "side_norm"] = get(c + "side.gate"), get(c + "side.proj"), get(c + "side.norm")
        W[p + "w_in"] = w_in
    out = {}
    for k, v in W.items():
        f32 = k.rsplit(".", 1)[-1] in _SUVAPEL_F32
        out[k] = v.to(device=device, dtype=torch.float32 if f32 else dtype).contiguous()
    return out


def suvapel_check_shapes(cfg, W: Dict[str, torch.Tensor]) -> None:
    """Every tensor of the engine layout has the shape the configuration implies (the low-rank pairs' inner sizes
    are the tensors' own)."""
    h, V = cfg.hidden, cfg.vocab_size
    want = {"embed": (V, h), "lm_head": (V, h), "norm_w": (h,), "norm_b": (h,), "norm_alpha": (1,)}
    if cfg.side_dim:
        want["side_embed"] = (V, cfg.side_dim * cfg.num_layers)
    for i, L in enumerate(cfg.layers):
        p, m, a = f"layers.{i}.", L.delta, L.attention
        ra = W[p + "w_a2"].shape[1] if p + "w_a2" in W else 0
        rg = W[p + "w_g2"].shape[1] if p + "w_g2" in W else 0
        want.update({p + "norm_w": (h,), p + "norm_b": (h,), p + "norm_alpha": (1,),
                     p + "w_in": (suvapel_columns(L, ra, rg)["total"], h), p + "conv": (m.conv, m.conv_channels()),
                     p + "A_log": (m.heads,), p + "dt_bias": (m.heads * m.dim if m.channel_decay else m.heads,),
                     p + "hnorm": (m.heads * m.vdim,), p + "wo": (h, m.heads * m.vdim)})
        if m.channel_decay:
            want.update({p + "w_a2": (m.heads * m.dim, ra), p + "w_g2": (m.heads * m.vdim, rg)})
        if a is not None:
            want.update({p + "att_conv": (a.conv, a.heads * a.dim + a.kv_heads * (a.dim + a.vdim)),
                         p + "att_wo": (h, a.heads * a.vdim), p + "inv_freq": (a.rot.dims // 2,)})
        if L.ff:
            want.update({p + "b_gu": (2 * L.ff,), p + "w_down": (h, L.ff), p + "b_down": (h,)})
        if cfg.side_dim:
            want.update({p + "side_gate": (cfg.side_dim, h), p + "side_proj": (h, cfg.side_dim), p + "side_norm": (h,)})
    for k, shp in want.items():
        if k not in W or tuple(W[k].shape) != shp:
            raise ValueError(f"tensor {k}: expected shape {shp}, found {tuple(W[k].shape) if k in W else None}")


def suvapel_checkpoint_tensors(cfg, seed: int = 0, dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """Random tensors under the checkpoint's own names (what a Suvapel model.safetensors holds)."""
    g = torch.Generator().manual_seed(_seed(seed, "suvapel") & 0x7FFFFFFF)
    h, V = cfg.hidden, cfg.vocab_size

    def mat(o, i, std=None):
        return (torch.randn(o, i, generator=g) * (std if std is not None else i ** -0.5)).to(dtype)

    def vec(n, lo=0.75, hi=1.25):
        return (lo + (hi - lo) * torch.rand(n, generator=g)).to(dtype)

    def dyt(name):
        return {name: vec(h), name + ".b": (torch.randn(h, generator=g) * 0.05).to(dtype),
                name + ".alpha": (0.4 + 0.4 * torch.rand((), generator=g)).to(dtype)}

    def conv(c, taps):
        w = torch.randn(c, taps, generator=g) * 0.3
        w[:, -1] += 1.0
        return w.to(dtype)

    T = {"embed": mat(V, h, 1.0), "head": mat(V, h), **dyt("final.norm")}
    if cfg.side_dim:
        T["side.embed"] = mat(V, cfg.side_dim * cfg.num_layers, 1.0)
    for i, L in enumerate(cfg.layers):
        c, m, a = f"l{i}.", L.delta, L.attention
        T.update(dyt(c + "norm1"))
        if a is not None:
            l = c + "mix.left."
            for k, n in (("q", a.heads * a.dim), ("k", a.kv_heads * a.dim), ("v", a.kv_heads * a.vdim)):
                T[l + k], T[l + k + ".conv"] = mat(n, h), conv(n, a.conv)
            T[l + "g"], T[l + "o"] = mat(a.heads, h), mat(h, a.heads * a.vdim)
        r = c + ("mix.right." if a is not None else "mix.")
        for k, n in (("q", m.kv_heads * m.dim), ("k", m.kv_heads * m.dim), ("v", m.heads * m.vdim)):
            T[r + k], T[r + k + ".conv"] = mat(n, h, 2.0 * h ** -0.5), conv(n, m.conv)
        T[r + "b"] = mat(m.heads, h)
        T[r + "A_log"] = torch.log(0.5 + 3.5 * torch.rand(m.heads, generator=g)).to(dtype)
        T[r + "norm"], T[r + "o"] = vec(m.vdim), mat(h, m.heads * m.vdim)
        if m.channel_decay:
            R = m.low_rank
            T[r + "a1"], T[r + "a2"] = mat(R, h), mat(m.heads * m.dim, R)
            T[r + "g1"], T[r + "g2"] = mat(R, h), mat(m.heads * m.vdim, R)
            T[r + "dt_bias"] = (torch.randn(m.heads * m.dim, generator=g) - 3.0).to(dtype)
        else:
            T[r + "a"], T[r + "g"] = mat(m.heads, h), mat(m.heads * m.vdim, h)
            T[r + "dt_bias"] = (torch.randn(m.heads, generator=g) - 3.0).to(dtype)
        if L.ff:
            for k, o_, i_ in (("gate", L.ff, h), ("up", L.ff, h), ("down", h, L.ff)):
                T[c + "mlp." + k] = mat(o_, i_)
                T[c + "mlp." + k + ".b"] = (torch.randn(o_, generator=g) * 0.1).to(dtype)
        if cfg.side_dim:
            T[c + "side.gate"], T[c + "side.proj"] = mat(cfg.side_dim, h), mat(h, cfg.side_dim)
            T[c + "side.norm"] = vec(h, 0.2, 0.6)
    return T


def suvapel_random_weights(cfg, seed: int = 0, device="cpu", dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """Random-init Suvapel weights: drawn in bf16 (as a checkpoint stores them), packed for `dtype`."""
    T = suvapel_checkpoint_tensors(cfg, seed)
    W = _suvapel_pack(cfg, T.__getitem__, device, dtype)
    suvapel_check_shapes(cfg, W)
    return W


def load_suvapel_safetensors(path: str, cfg, device="cpu", dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """A Suvapel checkpoint (a file, or a folder holding model.safetensors / *.safetensors)."""
    W = _suvapel_pack(cfg, _safetensors_getter(path), device, dtype)
    suvapel_check_shapes(cfg, W)
    return W


# ------------------------------------------------------------------------------------------------
# Zibinex.  Engine layout per layer that has tensors of its own, `layers.<i>.` (activation dtype unless marked fp32;
# a layer with weights_of has no entries, the model points it at its owner's):
#   norm1, norm1b, norm2, norm2b [W] fp32, kept as 1 + w (the checkpoint holds w, the offset from 1)
#   latent attention:  w_in [dkv rows (kv_rank + rot_dim); q rows (H * (dim + rot_dim)); g rows (H); zero rows up to a
#           multiple of 8, W] (one GEMM; `zibinex_columns`), kv_norm [kv_rank] fp32, w_uk [H, dim, kv_rank],
#           w_uv [H, vdim, kv_rank], wo [W, H * vdim] (the rotary table belongs to the layer's entry: the model makes it)
#   attention:  w_qkv [q; k; v rows, W] + b_qkv (one GEMM), q_norm / k_norm [dim] fp32, dist [3, H] fp32 (the rows
#           r1, r2, pb), wo [W, H * vdim]
#   dense feed-forward:  w_gu [gate rows; up rows, W], w_down [W, ff]
#   experts:  w_router [E, W] fp32, w_gu_e [E, 2 ff, W] (gate rows, then up rows), w_dn_e [E, W, ff]
# The LM head is the embedding table.
_ZIBINEX_F32 = ("norm1", "norm1b", "norm2", "norm2b", "kv_norm", "q_norm", "k_norm", "dist", "w_router")


def zibinex_columns(m) -> Dict[str, int]:
    """Column offsets of a latent-attention layer's fused input projection."""
    q = m.kv_rank + m.rot_dim
    g = q + m.heads * (m.dim + m.rot_dim)
    return {"kv": 0, "q": q, "g": g, "total": _pad8(g + m.heads)}


def _zibinex_pack(cfg, get, device, dtype) -> Dict[str, torch.Tensor]:
    def one_plus(name):
        return 1.0 + get(name).float()

    W: Dict[str, torch.Tensor] = {"embed": get("embed"), "norm": one_plus("final.norm")}
    for i, L in enumerate(cfg.layers):
        if L.weights_of >= 0:
            continue
        p, c, m, f = f"layers.{i}.", f"l{i}.", L.mixer, L.mlp
        for k in ("norm1", "norm1b") + (("norm2", "norm2b") if f is not None else ()):
            W[p + k] = one_plus(c + k)
        if m.kind == "latent_attention":
            rows = torch.cat([get(c + "mix.dkv"), get(c + "mix.q"), get(c + "mix.g")])
            pad = zibinex_columns(m)["total"] - rows.shape[0]
            W[p + "w_in"] = torch.cat([rows, rows.new_zeros((pad, rows.shape[1]))]) if pad else rows
            W[p + "kv_norm"] = get(c + "mix.dkv.norm")
            W[p + "w_uk"] = get(c + "mix.uk").view(m.heads, m.dim, m.kv_rank)
            W[p + "w_uv"] = get(c + "mix.uv").view(m.heads, m.vdim, m.kv_rank)
        else:
            W[p + "w_qkv"] = torch.cat([get(c + "mix.q"), get(c + "mix.k"), get(c + "mix.v")])
            W[p + "b_qkv"] = torch.cat([get(c + "mix.q.b"), get(c + "mix.k.b"), get(c + "mix.v.b")])
            W[p + "q_norm"], W[p + "k_norm"] = get(c + "mix.q.norm"), get(c + "mix.k.norm")
            W[p + "dist"] = torch.stack([get(c + "mix.r1"), get(c + "mix.r2"), get(c + "mix.pb")])
        W[p + "wo"] = get(c + "mix.o")
        if f is None:
            continue
        if f.kind == "dense":
            W[p + "w_gu"], W[p + "w_down"] = torch.cat([get(c + "mlp.gate"), get(c + "mlp.up")]), get(c + "mlp.down")
        else:
            W[p + "w_router"] = get(c + "mlp.router")
            W[p + "w_gu_e"] = torch.stack([torch.cat([get(c + f"mlp.e{e}.gate"), get(c + f"mlp.e{e}.up")])
                                           for e in range(f.experts)])
            W[p + "w_dn_e"] = torch.stack([get(c + f"mlp.e{e}.down") for e in range(f.experts)])
    out = {}
    for k, v in W.items():
        f32 = k == "norm" or k.rsplit(".", 1)[-1] in _ZIBINEX_F32
        out[k] = v.to(device=device, dtype=torch.float32 if f32 else dtype).contiguous()
    out["lm_head"] = out["embed"]
    return out


def zibinex_check_shapes(cfg, W: Dict[str, torch.Tensor]) -> None:
    """Every tensor of the engine layout has the shape the configuration implies."""
    h, V = cfg.hidden, cfg.vocab_size
    want = {"embed": (V, h), "norm": (h,)}
    for i, L in enumerate(cfg.layers):
        if L.weights_of >= 0:
            continue
        p, m, f = f"layers.{i}.", L.mixer, L.mlp
        want.update({p + "norm1": (h,), p + "norm1b": (h,), p + "wo": (h, m.heads * m.vdim)})
        if m.kind == "latent_attention":
            want.update({p + "w_in": (zibinex_columns(m)["total"], h), p + "kv_norm": (m.kv_rank,),
                         p + "w_uk": (m.heads, m.dim, m.kv_rank), p + "w_uv": (m.heads, m.vdim, m.kv_rank)})
        else:
            n = m.heads * m.dim + m.kv_heads * (m.dim + m.vdim)
            want.update({p + "w_qkv": (n, h), p + "b_qkv": (n,), p + "q_norm": (m.dim,), p + "k_norm": (m.dim,),
                         p + "dist": (3, m.heads)})
        if f is not None:
            want.update({p + "norm2": (h,), p + "norm2b": (h,)})
            if f.kind == "dense":
                want.update({p + "w_gu": (2 * f.ff, h), p + "w_down": (h, f.ff)})
            else:
                want.update({p + "w_router": (f.experts, h), p + "w_gu_e": (f.experts, 2 * f.ff, h),
                             p + "w_dn_e": (f.experts, h, f.ff)})
    for k, shp in want.items():
        if k not in W or tuple(W[k].shape) != shp:
            raise ValueError(f"tensor {k}: expected shape {shp}, found {tuple(W[k].shape) if k in W else None}")


def zibinex_checkpoint_tensors(cfg, seed: int = 0, dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """Random tensors under the checkpoint's own names (what a Zibinex model.safetensors holds)."""
    g = torch.Generator().manual_seed(_seed(seed, "zibinex") & 0x7FFFFFFF)
    h, V = cfg.hidden, cfg.vocab_size

    def mat(o, i, std=None):
        return (torch.randn(o, i, generator=g) * (std if std is not None else i ** -0.5)).to(dtype)

    def vec(n, lo=0.75, hi=1.25):
        return (lo + (hi - lo) * torch.rand(n, generator=g)).to(dtype)

    T = {"embed": mat(V, h, 1.0), "final.norm": vec(h, -0.25, 0.25)}
    for i, L in enumerate(cfg.layers):
        if L.weights_of >= 0:
            continue
        c, m, f = f"l{i}.", L.mixer, L.mlp
        for k in ("norm1", "norm1b") + (("norm2", "norm2b") if f is not None else ()):
            T[c + k] = vec(h, -0.25, 0.25)
        if m.kind == "latent_attention":
            T[c + "mix.q"] = mat(m.heads * (m.dim + m.rot_dim), h)
            T[c + "mix.dkv"], T[c + "mix.dkv.norm"] = mat(m.kv_rank + m.rot_dim, h), vec(m.kv_rank)
            T[c + "mix.uk"], T[c + "mix.uv"] = mat(m.heads * m.dim, m.kv_rank), mat(m.heads * m.vdim, m.kv_rank)
            T[c + "mix.g"] = mat(m.heads, h)
        else:
            for k, n in (("q", m.heads * m.dim), ("k", m.kv_heads * m.dim), ("v", m.kv_heads * m.vdim)):
                T[c + "mix." + k], T[c + f"mix.{k}.b"] = mat(n, h), (torch.randn(n, generator=g) * 0.1).to(dtype)
            T[c + "mix.q.norm"], T[c + "mix.k.norm"] = vec(m.dim), vec(m.dim)
            T[c + "mix.r1"], T[c + "mix.r2"] = vec(m.heads, 0.25, 1.0), vec(m.heads, 0.1, 1.0)
            T[c + "mix.pb"] = vec(m.heads, -3.0, -1.0)
        T[c + "mix.o"] = mat(h, m.heads * m.vdim)
        if f is not None and f.kind == "dense":
            T[c + "mlp.gate"], T[c + "mlp.up"], T[c + "mlp.down"] = mat(f.ff, h), mat(f.ff, h), mat(h, f.ff)
        elif f is not None:
            T[c + "mlp.router"] = mat(f.experts, h, 2.0 * h ** -0.5)
            for e in range(f.experts):
                n = f"mlp.e{e}."
                T[c + n + "gate"], T[c + n + "up"], T[c + n + "down"] = mat(f.ff, h), mat(f.ff, h), mat(h, f.ff)
    return T


def zibinex_random_weights(cfg, seed: int = 0, device="cpu", dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """Random-init Zibinex weights: drawn in bf16 (as a checkpoint stores them), packed for `dtype`."""
    T = zibinex_checkpoint_tensors(cfg, seed)
    W = _zibinex_pack(cfg, T.__getitem__, device, dtype)
    zibinex_check_shapes(cfg, W)
    return W


def load_zibinex_safetensors(path: str, cfg, device="cpu", dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """A Zibinex checkpoint (a file, or a folder holding model.safetensors / *.safetensors)."""
    W = _zibinex_pack(cfg, _safetensors_getter(path), device, dtype)
    zibinex_check_shapes(cfg, W)
    return W


def build_weights(spec: str, cfg: ModelConfig, par: ParallelInfo, device="cpu", dtype=torch.bfloat16):
    if getattr(cfg, "family", "") == "vivepel":
        if par.tp_size != 1 or par.ep_size != 1:
            raise ValueError("Vivepel runs at TP = 1 (data parallel replicas scale it out)")
        if spec.startswith("random"):
            seed = int(spec.split(":", 1)[1]) if ":" in spec else 0
            return vivepel_random_weights(cfg, seed=seed, device=device, dtype=dtype)
        return load_vivepel_safetensors(spec, cfg, device=device, dtype=dtype)
    if getattr(cfg, "family", "") == "kafilorn":
        if par.tp_size != 1 or par.ep_size != 1:
            raise ValueError("Kafilorn runs at TP = 1 (data parallel replicas scale it out)")
        if spec.startswith("random"):
            seed = int(spec.split(":", 1)[1]) if ":" in spec else 0
            return kafilorn_random_weights(cfg, seed=seed, device=device, dtype=dtype)
        return load_kafilorn_safetensors(spec, cfg, device=device, dtype=dtype)
    if getattr(cfg, "family", "") == "suvapel":
        if par.tp_size != 1 or par.ep_size != 1:
            raise ValueError("Suvapel runs at TP = 1 (data parallel replicas scale it out)")
        if spec.startswith("random"):
            seed = int(spec.split(":", 1)[1]) if ":" in spec else 0
            return suvapel_random_weights(cfg, seed=seed, device=device, dtype=dtype)
        return load_suvapel_safetensors(spec, cfg, device=device, dtype=dtype)
    if getattr(cfg, "family", "") == "zibinex":
        if par.tp_size != 1 or par.ep_size != 1:
            raise ValueError("Zibinex runs at TP = 1 (data parallel replicas scale it out)")
        if spec.startswith("random"):
            seed = int(spec.split(":", 1)[1]) if ":" in spec else 0
            return zibinex_random_weights(cfg, seed=seed, device=device, dtype=dtype)
        return load_zibinex_safetensors(spec, cfg, device=device, dtype=dtype)
    if spec.startswith("random"):
        seed = int(spec.split(":", 1)[1]) if ":" in spec else 0
        return random_weights(cfg, par, seed=seed, device=device, dtype=dtype)
    return load_safetensors(spec, cfg, par, device=device, dtype=dtype)
