"""A plain, slow Zibinex in float64 numpy: one function per mechanism, whole sequences recomputed from their first
token with no cache, written from the design's equations and sharing no code with the package.  Also the builders
of small configurations and random checkpoints that the tests use.

  norm(x; w)         x / sqrt(mean(x^2) + eps) * (1 + w)                      a checkpoint holds w, the offset from 1
  layer              x <- x + norm(mixer(norm(x; n1)); n1b);   x <- x + norm(ff(norm(x; n2)); n2b)
  latent attention   q_h = [q_h^n | q_h^r] rows of Wq h;  [c' | k^r] = Wdkv h;  c = c' / rms(c') * w_c
                     rotary on q_h^r and k^r, pairs (2i, 2i + 1), angle p f_i, cos and sin times a magnitude
                     s_h(i, j) = scale (q_h^n . Wuk_h c_j + q_h^r . k^r_j),  j <= i (and i - j < window, if any)
                     out = Wo [ sigmoid(Wg h)_h * sum_j softmax_j(s_h) Wuv_h c_j ]_h
  attention          q, k, v = W h + b;  q, k per head / rms * w (plain weight);  head h uses k / v head h // (H / G)
                     a_h(i, j) = sigmoid(scale q_h(i) . k(j) - r1_h ln(1 + r2_h (i - j)) + pb_h),  0 <= i - j < window
                     out = Wo [ sum_j a_h(i, j) v(j) ]_h                       the weights are not normalised
  dense              Wd (g sigmoid(1.702 g) (u + 1)),  g = min(Wg h, limit),  u = clamp(Wu h, -limit, limit)
  experts            s = sigmoid(Wr h);  the `top` largest s_e;  y = sum_e E_e(s_e h),  E(x) = Wd (silu(Wg x) * Wu x)
  logits             embed . norm(x; final)
A layer with weights_of = j computes with layer j's tensors and the constants of its own entry.
"""
import math

import numpy as np
import torch


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def rms_div(x, eps):
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps)


def norm_one_plus(x, w, eps):
    return rms_div(x, eps) * (1.0 + w)


def rotary_table(dims, base, scaling):
    """(frequencies [dims / 2], magnitude of cos and sin); scaling None or {factor, original, fast, slow}."""
    f = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)])
    if not scaling:
        return f, 1.0

    def turn_dim(turns):
        return dims * math.log(scaling["original"] / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(turn_dim(scaling["fast"])), 0)
    hi = min(math.ceil(turn_dim(scaling["slow"])), dims - 1)
    ramp = np.clip((np.arange(dims // 2) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / scaling["factor"] * ramp + f * (1.0 - ramp), 0.1 * math.log(scaling["factor"]) + 1.0


def rotate_pairs(x, pos, freq, mag, dims):
    """x [T, ..., n]: entries (2i, 2i + 1), i < dims / 2, turned by the angle pos * freq[i]; the rest unchanged."""
    out = np.array(x, dtype=np.float64)
    for t in range(x.shape[0]):
        for i in range(dims // 2):
            a = pos[t] * freq[i]
            c, s = math.cos(a) * mag, math.sin(a) * mag
            u, v = x[t, ..., 2 * i].copy(), x[t, ..., 2 * i + 1].copy()
            out[t, ..., 2 * i] = u * c - v * s
            out[t, ..., 2 * i + 1] = v * c + u * s
    return out


def softmax_attention(q, k, v, scale, window=0):
    """q, k [T, H, D], v [T, H, Dv]; causal, optionally 0 <= i - j < window.  -> [T, H, Dv]."""
    T, H, _ = q.shape
    out = np.zeros((T, H, v.shape[2]))
    for i in range(T):
        lo = max(0, i - window + 1) if window else 0
        for h in range(H):
            s = (k[lo:i + 1, h] @ q[i, h]) * scale
            w = np.exp(s - s.max())
            out[i, h] = (w / w.sum()) @ v[lo:i + 1, h]
    return out


def sigmoid_attention(q, k, v, scale, r1, r2, pb, window=0):
    """q [T, H, D], k [T, G, D], v [T, G, Dv]: weight of key j for query i is sigmoid(scale q . k - r1 ln(1 + r2 (i - j))
    + pb) for 0 <= i - j < window (window 0: every j <= i); no normalisation.  -> [T, H, Dv]."""
    T, H, _ = q.shape
    rep = H // k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    for i in range(T):
        lo = max(0, i - window + 1) if window else 0
        dist = i - np.arange(lo, i + 1)
        for h in range(H):
            s = (k[lo:i + 1, h // rep] @ q[i, h]) * scale - r1[h] * np.log(1.0 + r2[h] * dist) + pb[h]
            out[i, h] = sigmoid(s) @ v[lo:i + 1, h // rep]
    return out


def latent_mixer(h, m, A, p, eps):
    T = h.shape[0]
    H, Dn, Dr, Dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    q = (h @ A[p + "q"].T).reshape(T, H, Dn + Dr)
    dkv = h @ A[p + "dkv"].T
    c = rms_div(dkv[:, :R], eps) * A[p + "dkv.norm"]
    kr = dkv[:, R:]
    qr = q[:, :, Dn:]
    rot = m.get("rot")
    pos = np.arange(T)
    if rot:
        f, mag = rotary_table(rot["dims"], rot["base"], rot.get("scaling"))
        qr, kr = rotate_pairs(qr, pos, f, mag, rot["dims"]), rotate_pairs(kr, pos, f, mag, rot["dims"])
    kn = (c @ A[p + "uk"].T).reshape(T, H, Dn)
    v = (c @ A[p + "uv"].T).reshape(T, H, Dv)
    qf = np.concatenate([q[:, :, :Dn], qr], axis=2)
    kf = np.concatenate([kn, np.repeat(kr[:, None, :], H, axis=1)], axis=2)
    o = softmax_attention(qf, kf, v, m["scale"], (m.get("mask") or {}).get("size", 0))
    o = o * sigmoid(h @ A[p + "g"].T)[:, :, None]
    return o.reshape(T, H * Dv) @ A[p + "o"].T


def attention_mixer(h, m, A, p, eps):
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ A[p + "q"].T + A[p + "q.b"]).reshape(T, H, D)
    k = (h @ A[p + "k"].T + A[p + "k.b"]).reshape(T, G, D)
    v = (h @ A[p + "v"].T + A[p + "v.b"]).reshape(T, G, Dv)
    q, k = rms_div(q, eps) * A[p + "q.norm"], rms_div(k, eps) * A[p + "k.norm"]
    o = sigmoid_attention(q, k, v, m["scale"], A[p + "r1"], A[p + "r2"], A[p + "pb"], (m.get("mask") or {}).get("size", 0))
    return o.reshape(T, H * Dv) @ A[p + "o"].T


def dense_ff(h, f, A, p):
    g = np.minimum(h @ A[p + "gate"].T, f["limit"])
    u = np.clip(h @ A[p + "up"].T, -f["limit"], f["limit"])
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ A[p + "down"].T


def route(h, A, p, top):
    """-> (chosen experts [T, top], their scores [T, top]); ties go to the lower index."""
    s = sigmoid(h @ A[p + "router"].T)
    ids = np.argsort(-s, axis=-1, kind="stable")[:, :top]
    return ids, np.take_along_axis(s, ids, axis=-1)


def expert_ff(h, f, A, p):
    ids, w = route(h, A, p, f["router"]["top"])
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        for e, s in zip(ids[t], w[t]):
            x = s * h[t]
            out[t] += (silu(x @ A[p + f"e{e}.gate"].T) * (x @ A[p + f"e{e}.up"].T)) @ A[p + f"e{e}.down"].T
    return out


def forward(config, A, tokens, layer_out=None):
    """Logits [T, vocab] of a whole sequence; layer_out collects the residual after every layer."""
    eps = config["norm"]["eps"]
    x = A["embed"][np.asarray(tokens)]
    for i, L in enumerate(config["layers"]):
        p = "l%d." % L.get("weights_of", i)
        h = norm_one_plus(x, A[p + "norm1"], eps)
        mixer = latent_mixer if L["type"] == "latent_attention" else attention_mixer
        x = x + norm_one_plus(mixer(h, L["mixer"], A, p + "mix.", eps), A[p + "norm1b"], eps)
        f = L.get("mlp")
        if f:
            h = norm_one_plus(x, A[p + "norm2"], eps)
            y = dense_ff(h, f, A, p + "mlp.") if f["kind"] == "dense" else expert_ff(h, f, A, p + "mlp.")
            x = x + norm_one_plus(y, A[p + "norm2b"], eps)
        if layer_out is not None:
            layer_out.append(x.copy())
    return norm_one_plus(x, A["final.norm"], eps) @ A["embed"].T


def as_arrays(W):
    return {k: v.double().numpy() for k, v in W.items()}


# ---- small configurations --------------------------------------------------------------------------
def latent_layer(heads=3, dim=6, rot_dim=4, vdim=5, kv_rank=12, rot_dims=None, base=100.0, scaling=(4.0, 32, 8.0, 1.0),
                 scale=0.4, window=0, mlp="moe", **kw):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale}
    rd = rot_dim if rot_dims is None else rot_dims
    if rd:
        m["rot"] = {"dims": rd, "base": base}
        if scaling:
            m["rot"]["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    if window:
        m["mask"] = {"size": window}
    return {"type": "latent_attention", "mixer": m, "mlp": ff_cfg(mlp, **kw)}


def attention_layer(heads=4, kv_heads=2, dim=6, vdim=5, window=8, scale=0.5, mlp="moe", **kw):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window:
        m["mask"] = {"size": window}
    return {"type": "attention", "mixer": m, "mlp": ff_cfg(mlp, **kw)}


def ff_cfg(kind, ff=20, limit=0.75, experts=5, top=2):
    if kind is None:
        return None
    if kind == "dense":
        return {"kind": "dense", "ff": ff, "limit": limit}
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def shared(layer, owner):
    """A layer that runs on layer `owner`'s tensors (the sizes of its entry equal the owner's)."""
    return dict(layer, weights_of=owner)


def make_config(layers, width=24, vocab=64, eps=1e-5):
    return {"architecture": "Zibinex", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}


def random_tensors(config, seed=0, dtype=torch.bfloat16):
    """Random tensors under the checkpoint's names, rounded to bf16 (what a checkpoint stores) and returned as fp32."""
    g = torch.Generator().manual_seed(seed)
    W, h = {}, config["width"]

    def mat(o, i, std=None):
        return (torch.randn(o, i, generator=g) * (std if std is not None else i ** -0.5)).to(dtype).float()

    def vec(n, lo, hi):
        return (lo + (hi - lo) * torch.rand(n, generator=g)).to(dtype).float()

    W["embed"], W["final.norm"] = mat(config["vocab"], h, 1.0), vec(h, -0.4, 0.4)
    for i, L in enumerate(config["layers"]):
        if "weights_of" in L:
            continue
        c, m, f = "l%d." % i, L["mixer"], L.get("mlp")
        for k in ("norm1", "norm1b") + (("norm2", "norm2b") if f else ()):
            W[c + k] = vec(h, -0.4, 0.4)
        if L["type"] == "latent_attention":
            W[c + "mix.q"] = mat(m["heads"] * (m["dim"] + m["rot_dim"]), h, 2.0 * h ** -0.5)
            W[c + "mix.dkv"], W[c + "mix.dkv.norm"] = mat(m["kv_rank"] + m["rot_dim"], h), vec(m["kv_rank"], 0.5, 1.5)
            W[c + "mix.uk"] = mat(m["heads"] * m["dim"], m["kv_rank"])
            W[c + "mix.uv"] = mat(m["heads"] * m["vdim"], m["kv_rank"])
            W[c + "mix.g"] = mat(m["heads"], h, 2.0 * h ** -0.5)
        else:
            for k, n in (("q", m["heads"] * m["dim"]), ("k", m["kv_heads"] * m["dim"]), ("v", m["kv_heads"] * m["vdim"])):
                W[c + "mix." + k] = mat(n, h)
                W[c + "mix." + k + ".b"] = (torch.randn(n, generator=g) * 0.3).to(dtype).float()
            W[c + "mix.q.norm"], W[c + "mix.k.norm"] = vec(m["dim"], 0.5, 2.0), vec(m["dim"], 0.5, 2.0)
            W[c + "mix.r1"], W[c + "mix.r2"] = vec(m["heads"], 0.2, 1.5), vec(m["heads"], 0.1, 2.0)
            W[c + "mix.pb"] = vec(m["heads"], -2.5, 0.5)
        W[c + "mix.o"] = mat(h, m["heads"] * m["vdim"])
        if f and f["kind"] == "dense":
            W[c + "mlp.gate"], W[c + "mlp.up"], W[c + "mlp.down"] = mat(f["ff"], h, 1.5 * h ** -0.5), mat(f["ff"], h, 1.5 * h ** -0.5), mat(h, f["ff"])
        elif f:
            W[c + "mlp.router"] = mat(f["router"]["experts"], h, 2.0 * h ** -0.5)
            for e in range(f["router"]["experts"]):
                n = c + "mlp.e%d." % e
                W[n + "gate"], W[n + "up"], W[n + "down"] = mat(f["expert"]["ff"], h), mat(f["expert"]["ff"], h), mat(h, f["expert"]["ff"])
    return W
