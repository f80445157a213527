"""A plain, slow Suvapel in float64 numpy: one function per mechanism, whole sequences recomputed from their first
token, no cache, no state object, no code shared with the package.  Tests compare the engine with it.

Notation: x the residual row [W]; h the normed row; t a position counted from 0; W_foo the tensor
'<layer>.mix.foo' (or '<layer>.mlp.foo'), stored [out, in].
"""
from __future__ import annotations

import json
import math
import os

import numpy as np


# ---- elementwise --------------------------------------------------------------------------------------
def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rms_div(v, eps):
    return v / np.sqrt(np.mean(v * v, axis=-1, keepdims=True) + eps)


def dyt(x, alpha, w, b):
    """Dynamic Tanh: no statistics, a learned slope, weight and bias."""
    return np.tanh(alpha * x) * w + b


# ---- short causal convolution --------------------------------------------------------------------------
def short_conv(u, w):
    """u [T, C], w [C, taps]; the last column of w meets the current row, rows before the start are zero."""
    T, C = u.shape
    taps = w.shape[1]
    y = np.zeros_like(u)
    for t in range(T):
        for j in range(taps):
            s = t - (taps - 1) + j
            if s >= 0:
                y[t] += w[:, j] * u[s]
    return y


# ---- rotary positions with YaRN-scaled frequencies -----------------------------------------------------
def rotary_table(dims, base, scaling):
    """-> (frequencies [dims / 2], magnitude factor for cos and sin)."""
    half = dims // 2
    f = np.array([base ** (-2.0 * i / dims) for i in range(half)])
    if not scaling:
        return f, 1.0
    factor, orig = float(scaling["factor"]), float(scaling["original"])

    def turn_dim(turns):
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(turn_dim(float(scaling["fast"]))), 0)
    hi = min(math.ceil(turn_dim(float(scaling["slow"]))), dims - 1)
    ramp = np.clip((np.arange(half) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate(x, pos, freqs, mag):
    """x [heads, dim]: the first 2 * len(freqs) entries of each head rotated, pairs (i, i + half)."""
    half = len(freqs)
    out = x.copy()
    a = pos * freqs
    c, s = np.cos(a) * mag, np.sin(a) * mag
    u, v = x[:, :half], x[:, half:2 * half]
    out[:, :half] = u * c - v * s
    out[:, half:2 * half] = v * c + u * s
    return out


# ---- attention with a sliding window that keeps the first tokens ---------------------------------------
def visible(i, j, window, keep_first):
    return j <= i and (i - j < window or j < keep_first)


def window_attention(q, k, v, scale, window, keep_first):
    """q [T, H, D], k [T, G, D], v [T, G, Dv] -> [T, H, Dv]; softmax over the visible keys."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    for i in range(T):
        js = [j for j in range(i + 1) if visible(i, j, window, keep_first)]
        for h in range(H):
            g = h // (H // G)
            s = np.array([q[i, h] @ k[j, g] for j in js]) * scale
            w = np.exp(s - s.max())
            w /= w.sum()
            out[i, h] = sum(wj * v[j, g] for wj, j in zip(w, js))
    return out


def gated_attention(h, P, m, eps):
    """The attention mixer of a 'parallel' layer.  P: the mixer's tensors by their short names."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = short_conv(h @ P["q"].T, P["q.conv"]).reshape(T, H, D)
    k = short_conv(h @ P["k"].T, P["k.conv"]).reshape(T, G, D)
    v = short_conv(h @ P["v"].T, P["v.conv"]).reshape(T, G, Dv)
    rot = m.get("rot")
    if rot:
        freqs, mag = rotary_table(int(rot["dims"]), float(rot["base"]), rot.get("scaling"))
        q = np.stack([rotate(q[t], t, freqs, mag) for t in range(T)])
        k = np.stack([rotate(k[t], t, freqs, mag) for t in range(T)])
    mask = m.get("mask") or {}
    window = int(mask.get("size") or (T + 1))
    o = window_attention(q, k, v, float(m["scale"]), window, int(mask.get("keep_first") or 0))
    o = o * sigmoid(h @ P["g"].T)[:, :, None]
    return o.reshape(T, H * Dv) @ P["o"].T


# ---- gated delta rule ----------------------------------------------------------------------------------
def delta_rule(q, k, v, beta, decay):
    """q, k [T, H, D] (unit keys), v [T, H, Dv], beta [T, H], decay [T, H, D] (per key channel; a per-head decay is
    the same number in every channel) -> read-outs [T, H, Dv].  The memory starts at zero."""
    T, H, D = q.shape
    Dv = v.shape[2]
    out = np.zeros((T, H, Dv))
    for h in range(H):
        S = np.zeros((D, Dv))
        for t in range(T):
            S = decay[t, h][:, None] * S
            u = beta[t, h] * (v[t, h] - S.T @ k[t, h])
            S = S + np.outer(k[t, h], u)
            out[t, h] = S.T @ q[t, h]
    return out


def delta_mixer(h, P, m, eps, channel_decay):
    """channel_decay False: the 'delta' mixer (one decay per head, silu gate).  True: the recurrent half of a
    'parallel' mixer (one decay per head and key channel through a low-rank pair, sigmoid gate through another)."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_conv(h @ P["q"].T, P["q.conv"])).reshape(T, G, D)
    k = silu(short_conv(h @ P["k"].T, P["k.conv"])).reshape(T, G, D)
    v = silu(short_conv(h @ P["v"].T, P["v.conv"])).reshape(T, H, Dv)
    q = q / np.sqrt((q * q).sum(-1, keepdims=True) + 1e-6) * D ** -0.5
    k = k / np.sqrt((k * k).sum(-1, keepdims=True) + 1e-6)
    rep = H // G
    q, k = np.repeat(q, rep, axis=1), np.repeat(k, rep, axis=1)
    beta = sigmoid(h @ P["b"].T)
    if channel_decay:
        a = (h @ P["a1"].T) @ P["a2"].T + P["dt_bias"]
        decay = np.exp(-np.exp(P["A_log"])[None, :, None] * softplus(a).reshape(T, H, D))
        gate = sigmoid((h @ P["g1"].T) @ P["g2"].T)
    else:
        a = h @ P["a"].T + P["dt_bias"]
        decay = np.repeat(np.exp(-np.exp(P["A_log"])[None, :] * softplus(a))[:, :, None], D, axis=2)
        gate = silu(h @ P["g"].T)
    o = delta_rule(q, k, v, beta, decay)
    o = rms_div(o, eps) * P["norm"][None, None, :] * gate.reshape(T, H, Dv)
    return o.reshape(T, H * Dv) @ P["o"].T


# ---- feed-forward, token side input --------------------------------------------------------------------
def gated_ff(h, P):
    return (silu(h @ P["gate"].T + P["gate.b"]) * (h @ P["up"].T + P["up.b"])) @ P["down"].T + P["down.b"]


def token_side(x, tokens, table, layer, dim, P, eps):
    """The per-layer token input: a slice of a second embedding, gated by the residual, projected and RMS-normed."""
    e = table[tokens][:, layer * dim:(layer + 1) * dim]
    y = (gelu_tanh(x @ P["gate"].T) * e) @ P["proj"].T
    return rms_div(y, eps) * P["norm"]


# ---- the model -----------------------------------------------------------------------------------------
def sub(T, prefix):
    return {k[len(prefix):]: v for k, v in T.items() if k.startswith(prefix)}


def forward(cfg: dict, T: dict, tokens, layer_out=None):
    """cfg: config.json as a dict; T: tensors by checkpoint name (float64 arrays).  -> logits [len(tokens), vocab].
    layer_out: a list that receives the residual after every layer."""
    tokens = np.asarray(tokens, dtype=np.int64)
    eps, mult = float(cfg["norm"]["eps"]), float(cfg.get("residual_mult", 1.0))
    side = cfg.get("token_side")
    x = T["embed"][tokens]
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = dyt(x, T[p + "norm1.alpha"], T[p + "norm1"], T[p + "norm1.b"])
        m = L["mixer"]
        if L["type"] == "delta":
            y = delta_mixer(h, sub(T, p + "mix."), m, eps, False)
        elif L["type"] == "parallel":
            y = (float(m["left_scale"]) * gated_attention(h, sub(T, p + "mix.left."), m["left"], eps) +
                 float(m["right_scale"]) * delta_mixer(h, sub(T, p + "mix.right."), m["right"], eps, True))
        else:
            raise ValueError(L["type"])
        if L.get("mlp") is not None:
            y = y + gated_ff(h, sub(T, p + "mlp."))
        x = x + mult * y
        if side:
            x = x + mult * token_side(x, tokens, T["side.embed"], i, int(side["dim"]), sub(T, p + "side."), eps)
        if layer_out is not None:
            layer_out.append(x.copy())
    xf = dyt(x, T["final.norm.alpha"], T["final.norm"], T["final.norm.b"])
    return xf @ T["head"].T


def load_checkpoint(path: str):
    """config.json and model.safetensors of a folder -> (dict, float64 arrays); the file is parsed here, by hand."""
    with open(os.path.join(path, "config.json")) as f:
        cfg = json.load(f)
    with open(os.path.join(path, "model.safetensors"), "rb") as f:
        n = int.from_bytes(f.read(8), "little")
        head = json.loads(f.read(n))
        data = f.read()
    T = {}
    for name, e in head.items():
        if name == "__metadata__":
            continue
        lo, hi = e["data_offsets"]
        raw = data[lo:hi]
        if e["dtype"] == "BF16":
            a = (np.frombuffer(raw, dtype="<u2").astype(np.uint32) << 16).view(np.float32)
        elif e["dtype"] == "F32":
            a = np.frombuffer(raw, dtype="<f4")
        elif e["dtype"] == "I32":
            a = np.frombuffer(raw, dtype="<i4")
        else:
            raise ValueError(e["dtype"])
        T[name] = a.astype(np.float64).reshape(e["shape"])
    return cfg, T


# ---- small configurations and random checkpoints for the tests -----------------------------------------
def delta_mixer_cfg(heads=2, kv_heads=1, dim=8, vdim=12, conv=4):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}


def attention_cfg(heads=4, kv_heads=2, dim=16, vdim=8, conv=2, window=8, keep_first=2, rot_dims=8, base=50000.0,
                  scaling=(4.0, 64, 8.0, 2.0), scale=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv,
         "scale": scale if scale is not None else dim ** -0.5}
    if window:
        m["mask"] = {"size": window, "keep_first": keep_first}
    if rot_dims:
        m["rot"] = {"base": base, "dims": rot_dims}
        if scaling:
            m["rot"]["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return m


def delta_layer(ff=24, **kw):
    return {"type": "delta", "mixer": delta_mixer_cfg(**kw), "mlp": {"kind": "dense", "ff": ff} if ff else None}


def parallel_layer(left=None, right=None, left_scale=0.75, right_scale=1.1, ff=24):
    return {"type": "parallel", "mixer": {"left": left or attention_cfg(), "right": right or delta_mixer_cfg(conv=3),
                                          "left_scale": left_scale, "right_scale": right_scale},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def make_config(layers, width=32, vocab=96, side=6, mult=0.8, eps=1e-6):
    c = {"architecture": "Suvapel", "vocab": vocab, "width": width, "norm": {"eps": eps}, "residual_mult": mult,
         "layers": layers}
    if side:
        c["token_side"] = {"dim": side}
    return c


def random_tensors(cfg, seed=0, rank=5):
    """Random checkpoint tensors for `cfg` as torch bf16 tensors (what a checkpoint stores)."""
    import torch

    g = torch.Generator().manual_seed(seed)
    h, V = cfg["width"], cfg["vocab"]
    bf = torch.bfloat16

    def mat(o, i, std=None):
        return (torch.randn(o, i, generator=g) * (std if std is not None else i ** -0.5)).to(bf)

    def vec(n, lo=0.7, hi=1.3):
        return (lo + (hi - lo) * torch.rand(n, generator=g)).to(bf)

    def norm(name):
        return {name: vec(h), name + ".b": (torch.randn(h, generator=g) * 0.1).to(bf),
                name + ".alpha": (0.3 + 0.5 * torch.rand((), generator=g)).to(bf)}

    def conv(c, taps):
        return (torch.randn(c, taps, generator=g) * 0.5 + torch.eye(taps)[-1] * 0.8).to(bf)

    def delta(p, m, channel):
        H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        T = {}
        for k, n in (("q", G * D), ("k", G * D), ("v", H * Dv)):
            T[p + k], T[p + k + ".conv"] = mat(n, h, 2.0 * h ** -0.5), conv(n, m["conv"])
        T[p + "b"] = mat(H, h, 2.0 * h ** -0.5)
        T[p + "A_log"] = torch.log(0.3 + 4.0 * torch.rand(H, generator=g)).to(bf)
        T[p + "norm"], T[p + "o"] = vec(Dv), mat(h, H * Dv)
        if channel:
            T[p + "a1"], T[p + "a2"] = mat(rank, h), mat(H * D, rank, 2.0 * rank ** -0.5)
            T[p + "g1"], T[p + "g2"] = mat(rank + 2, h), mat(H * Dv, rank + 2, 2.0 * rank ** -0.5)
            T[p + "dt_bias"] = (torch.randn(H * D, generator=g) - 2.0).to(bf)
        else:
            T[p + "a"], T[p + "g"] = mat(H, h, 2.0 * h ** -0.5), mat(H * Dv, h)
            T[p + "dt_bias"] = (torch.randn(H, generator=g) - 2.0).to(bf)
        return T

    T = {"embed": mat(V, h, 1.0), "head": mat(V, h), **norm("final.norm")}
    side = (cfg.get("token_side") or {}).get("dim", 0)
    if side:
        T["side.embed"] = mat(V, side * len(cfg["layers"]), 1.0)
    for i, L in enumerate(cfg["layers"]):
        c, m = f"l{i}.", L["mixer"]
        T.update(norm(c + "norm1"))
        if L["type"] == "delta":
            T.update(delta(c + "mix.", m, False))
        else:
            a = m["left"]
            for k, n in (("q", a["heads"] * a["dim"]), ("k", a["kv_heads"] * a["dim"]), ("v", a["kv_heads"] * a["vdim"])):
                T[c + "mix.left." + k] = mat(n, h, 2.0 * h ** -0.5)
                T[c + "mix.left." + k + ".conv"] = conv(n, a["conv"])
            T[c + "mix.left.g"], T[c + "mix.left.o"] = mat(a["heads"], h, 2.0 * h ** -0.5), mat(h, a["heads"] * a["vdim"])
            T.update(delta(c + "mix.right.", m["right"], True))
        if L.get("mlp") is not None:
            ff = L["mlp"]["ff"]
            for k, o_, i_ in (("gate", ff, h), ("up", ff, h), ("down", h, ff)):
                T[c + "mlp." + k] = mat(o_, i_)
                T[c + "mlp." + k + ".b"] = (torch.randn(o_, generator=g) * 0.2).to(bf)
        if side:
            T[c + "side.gate"], T[c + "side.proj"] = mat(side, h), mat(h, side)
            T[c + "side.norm"] = vec(h, 0.2, 0.6)
    return T


def as_arrays(T):
    """torch tensors -> float64 numpy (what `forward` takes)."""
    return {k: v.double().numpy() for k, v in T.items()}
