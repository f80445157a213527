"""Model architecture presets (public HF configs; SURVEY.md §2.4 'Model constants').

The reference has no model code at all — its model is remote (`/root/reference/app.py:117`).
These are the architectures BASELINE.json names for the on-node engine, plus tiny variants of the
same shape family used by CPU tests and GPU numerics tests.
"""
from __future__ import annotations

import dataclasses
import json
import os
from typing import Dict, Optional, Tuple


@dataclasses.dataclass(frozen=True)
class ModelConfig:
    name: str
    family: str                 # "llama" | "mixtral"
    num_layers: int
    hidden: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    intermediate: int
    vocab_size: int
    rope_theta: float
    norm_eps: float = 1e-5
    max_position: int = 8192
    num_experts: int = 0        # mixtral
    top_k: int = 0
    tie_embeddings: bool = False
    tokenizer: str = "llama3"   # "llama3" | "llama2"

    @property
    def q_size(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_kv_heads * self.head_dim

    @property
    def qkv_size(self) -> int:
        return self.q_size + 2 * self.kv_size

    @property
    def is_moe(self) -> bool:
        return self.num_experts > 0

    def num_params(self) -> int:
        h, i, v = self.hidden, self.intermediate, self.vocab_size
        attn = h * self.qkv_size + self.q_size * h
        mlp = 3 * h * i * (self.num_experts if self.is_moe else 1) + (h * self.num_experts if self.is_moe else 0)
        per_layer = attn + mlp + 2 * h
        return self.num_layers * per_layer + v * h * (1 if self.tie_embeddings else 2) + h

    def default_step_tokens(self) -> int:
        """Engine token budget per step when MAX_NUM_BATCHED_TOKENS is 0 (auto).  Each step streams
        every weight once, so a step has a fixed cost that grows with the model: for an 8B model a
        256-request wave's ~8k prompt tokens are best split over ~3 mixed steps that also carry the
        running decodes (4096: 1243-1273 vs 1109-1122 req/s at 16384), while Mixtral-8x7B and
        Llama-3-70B do better with the wave's prompt in one step (16384: 269 vs 252 and 102 vs 91
        req/s; profiles/r2/budget/)."""
        return 4096 if self.num_params() * 2 < (40 << 30) else 16384

    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        return self.num_layers * 2 * self.kv_size * dtype_bytes


@dataclasses.dataclass(frozen=True)
class AttentionSpec:
    """One attention mixer of a per-layer-configured model (the `mixer` entry of a Vivepel layer)."""
    heads: int
    kv_heads: int
    dim: int                    # per-head query / key size
    vdim: int                   # per-head value size (the values are the projected keys: vdim == dim)
    chunk: int                  # chunked causal mask: position p sees floor(p / chunk) * chunk .. p (0: all of 0 .. p)
    rot_dims: int               # rotary positions on the first rot_dims entries of each head
    rot_base: float
    scale: float
    softcap: float

    @classmethod
    def from_dict(cls, m: dict) -> "AttentionSpec":
        mask, rot, cap = m.get("mask"), m.get("rot"), m.get("softcap")
        spec = cls(heads=int(m["heads"]), kv_heads=int(m["kv_heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                   chunk=int(mask["size"]) if mask else 0,            # no mask entry: plain causal
                   rot_dims=int(rot["dims"]) if rot else 0,           # no rot entry: no rotary positions
                   rot_base=float(rot["base"]) if rot else 1.0,
                   scale=float(m["scale"]), softcap=float(cap) if cap else 0.0)   # no softcap: scores as they are
        if spec.heads % spec.kv_heads:
            raise ValueError(f"heads {spec.heads} must be a multiple of kv_heads {spec.kv_heads}")
        if spec.vdim != spec.dim:
            raise ValueError(f"vdim {spec.vdim} != dim {spec.dim}: the values are the projected keys")
        if spec.rot_dims % 2 or spec.rot_dims > spec.dim or spec.chunk < 0:
            raise ValueError(f"bad rotary dims {spec.rot_dims} / chunk {spec.chunk} for head size {spec.dim}")
        return spec


@dataclasses.dataclass(frozen=True)
class LayerSpec:
    mixer: AttentionSpec
    ff: int = 0                 # dense feed-forward width; 0: the layer has no feed-forward


@dataclasses.dataclass(frozen=True)
class VivepelConfig:
    """Vivepel: a decoder whose layers are listed one by one in its config.json.  Every layer is
    x += ls1 * gnorm(mixer(gnorm(x))), then (if it has one) x += ls2 * gnorm(ff(gnorm(x))), with RMS
    norms in `norm_groups` groups; the mixer is chunk-masked attention (AttentionSpec), the
    feed-forward is up -> PolyNorm -> down.  The residual stream is fp32."""
    name: str
    vocab_size: int
    hidden: int
    norm_eps: float
    norm_groups: int
    layers: Tuple[LayerSpec, ...]
    max_position: int = 1 << 20
    tokenizer: str = "llama3"
    family: str = "vivepel"
    tie_embeddings: bool = False
    is_moe: bool = False

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, d: dict, name: str = "vivepel") -> "VivepelConfig":
        layers = []
        for i, L in enumerate(d["layers"]):
            if L["type"] != "attention":
                raise ValueError(f"layer {i}: unknown mixer type {L['type']!r}")
            mlp = L.get("mlp")
            if mlp is not None and mlp.get("kind") != "dense":
                raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
            layers.append(LayerSpec(AttentionSpec.from_dict(L["mixer"]), int(mlp["ff"]) if mlp is not None else 0))
        cfg = cls(name=name, vocab_size=int(d["vocab"]), hidden=int(d["width"]), norm_eps=float(d["norm"]["eps"]),
                  norm_groups=int(d["norm"]["groups"]), layers=tuple(layers))
        if cfg.hidden % cfg.norm_groups:
            raise ValueError(f"width {cfg.hidden} is not a multiple of norm groups {cfg.norm_groups}")
        return cfg

    def to_dict(self) -> dict:
        """The config.json form (what `from_dict` reads)."""
        return {"architecture": "Vivepel", "vocab": self.vocab_size, "width": self.hidden,
                "norm": {"eps": self.norm_eps, "groups": self.norm_groups},
                "layers": [{"type": "attention",
                            "mixer": {"heads": L.mixer.heads, "kv_heads": L.mixer.kv_heads, "dim": L.mixer.dim,
                                      "vdim": L.mixer.vdim, "mask": {"size": L.mixer.chunk} if L.mixer.chunk else None,
                                      "rot": {"base": L.mixer.rot_base, "dims": L.mixer.rot_dims},
                                      "scale": L.mixer.scale, "softcap": L.mixer.softcap},
                            "mlp": {"kind": "dense", "ff": L.ff} if L.ff else None} for L in self.layers]}

    def num_params(self) -> int:
        h = self.hidden
        n = 2 * self.vocab_size * h + h
        for L in self.layers:
            m = L.mixer
            n += (m.heads + m.kv_heads) * m.dim * (h + 1) + m.heads * m.vdim * h + m.heads * m.heads + 2 * m.dim + 3 * h
            if L.ff:
                n += 2 * h * L.ff + 4 + 3 * h
        return n

    def default_step_tokens(self) -> int:
        """16384: the tile attention kernel runs one workgroup per 16 query rows and CU, longest first; a
        step needs several times 256 of them for the causal tiles' unequal lengths to even out."""
        return 16384

    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        return sum(2 * L.mixer.kv_heads * L.mixer.dim * dtype_bytes for L in self.layers)


def vivepel_uniform(name: str, layers: int, hidden: int, heads: int, kv_heads: int, dim: int, ff: int, vocab: int,
                    chunk: int = 1024, rot_dims: Optional[int] = None, groups: int = 4) -> VivepelConfig:
    """A Vivepel configuration whose layers are all alike (benchmarks, tests)."""
    spec = AttentionSpec(heads, kv_heads, dim, dim, chunk, rot_dims if rot_dims is not None else dim // 2, 10000.0,
                         dim ** -0.5, 30.0)
    return VivepelConfig(name, vocab, hidden, 1e-6, groups, tuple(LayerSpec(spec, ff) for _ in range(layers)))


# ------------------------------------------------------------------------------------------------
# Kafilorn: layers listed one by one; a layer's mixer is an mLSTM (recurrent matrix memory, state slots)
# or latent attention (a low-rank key/value latent in the paged cache, sliding window, softmax sink,
# optionally borrowing another layer's cache); its feed-forward is dense (squared ReLU), a mixture of
# gated experts with a group-limited router, or absent; the residual is `streams` hyper-connected copies.
@dataclasses.dataclass(frozen=True)
class MLSTMSpec:
    """Matrix-memory recurrent mixer: per head a [dim, vdim] state, a normaliser [dim] and a running maximum."""
    heads: int
    dim: int
    vdim: int
    gate_cap: float             # gate pre-activations pass through cap * tanh(. / cap); 0: uncapped
    kind: str = "mlstm"

    @classmethod
    def from_dict(cls, m: dict) -> "MLSTMSpec":
        return cls(heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]), gate_cap=float(m.get("gate_cap") or 0.0))

    def to_dict(self) -> dict:
        d = {"heads": self.heads, "dim": self.dim, "vdim": self.vdim}
        if self.gate_cap:
            d["gate_cap"] = self.gate_cap
        return d

    def state_floats(self) -> int:
        return self.heads * (self.dim * self.vdim + self.dim + 1)


@dataclasses.dataclass(frozen=True)
class LatentAttentionSpec:
    """Attention whose keys and values are up-projections of a cached latent [kv_rank] plus one rotated key
    part [rot_dim] shared by all heads; queries come through a latent of their own [q_rank]."""
    heads: int
    dim: int                    # unrotated query / key entries per head
    rot_dim: int                # rotated query / key entries per head (the key part is shared by the heads)
    vdim: int
    q_rank: int
    kv_rank: int
    window: int                 # position i sees j with 0 <= i - j < window (0: all of 0 .. i)
    rot_dims: int               # rotary on the first rot_dims entries of the rotated part
    rot_base: float
    scale: float
    kv_from: int = -1           # >= 0: no key/value down-projection of its own, reads that layer's cache
    kind: str = "latent_attention"

    @classmethod
    def from_dict(cls, m: dict) -> "LatentAttentionSpec":
        mask, rot = m.get("mask"), m.get("rot")
        kv_from = m.get("kv_from")
        spec = cls(heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=int(m["rot_dim"]), vdim=int(m["vdim"]),
                   q_rank=int(m["q_rank"]), kv_rank=int(m["kv_rank"]), window=int(mask["size"]) if mask else 0,
                   rot_dims=int(rot["dims"]) if rot else 0, rot_base=float(rot["base"]) if rot else 1.0,
                   scale=float(m["scale"]), kv_from=-1 if kv_from is None else int(kv_from))
        if spec.rot_dims % 2 or spec.rot_dims > spec.rot_dim or spec.window < 0:
            raise ValueError(f"bad rotary dims {spec.rot_dims} / window {spec.window} for rotated size {spec.rot_dim}")
        return spec

    def to_dict(self) -> dict:
        d = {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim, "q_rank": self.q_rank,
             "kv_rank": self.kv_rank, "scale": self.scale}
        if self.window:
            d["mask"] = {"size": self.window}
        if self.rot_dims:
            d["rot"] = {"base": self.rot_base, "dims": self.rot_dims}
        if self.kv_from >= 0:
            d["kv_from"] = self.kv_from
        return d


@dataclasses.dataclass(frozen=True)
class FeedForwardSpec:
    """dense: down(relu(up h)^2), width ff.  moe: `experts` gated experts of width ff, `top` per token chosen
    among the best `keep_groups` of `groups` groups of neighbouring experts, plus a shared gated expert of
    width shared_ff for every token (0: none)."""
    kind: str                   # "dense" | "moe"
    ff: int
    experts: int = 0
    top: int = 0
    groups: int = 1
    keep_groups: int = 1
    shared_ff: int = 0

    @classmethod
    def from_dict(cls, m: dict) -> "FeedForwardSpec":
        if m["kind"] == "dense":
            return cls("dense", int(m["ff"]))
        if m["kind"] != "moe":
            raise ValueError(f"unknown feed-forward kind {m['kind']!r}")
        r, g, sh = m["router"], m["router"].get("groups"), m.get("shared")
        spec = cls("moe", int(m["expert"]["ff"]), experts=int(r["experts"]), top=int(r["top"]),
                   groups=int(g["count"]) if g else 1, keep_groups=int(g["keep"]) if g else 1,
                   shared_ff=int(sh["ff"]) if sh else 0)
        if spec.experts % spec.groups or not 0 < spec.keep_groups <= spec.groups or not 0 < spec.top <= spec.experts:
            raise ValueError(f"bad router: {spec}")
        if spec.top > spec.keep_groups * (spec.experts // spec.groups):
            raise ValueError(f"router: top {spec.top} exceeds the experts of {spec.keep_groups} groups")
        return spec

    def to_dict(self) -> dict:
        if self.kind == "dense":
            return {"kind": "dense", "ff": self.ff}
        r = {"experts": self.experts, "top": self.top}
        if self.groups > 1:
            r["groups"] = {"count": self.groups, "keep": self.keep_groups}
        d = {"kind": "moe", "expert": {"ff": self.ff}, "router": r}
        if self.shared_ff:
            d["shared"] = {"ff": self.shared_ff}
        return d


@dataclasses.dataclass(frozen=True)
class KafilornLayer:
    mixer: object               # MLSTMSpec | LatentAttentionSpec
    mlp: Optional[FeedForwardSpec]


_KAFILORN_MIXERS = {"mlstm": MLSTMSpec, "latent_attention": LatentAttentionSpec}


@dataclasses.dataclass(frozen=True)
class KafilornConfig:
    name: str
    vocab_size: int
    hidden: int
    norm_eps: float
    streams: int                # hyper-connection streams; 0: a plain residual sum
    embed_scale: float
    logit_scale: float
    layers: Tuple[KafilornLayer, ...]
    max_position: int = 1 << 20
    tokenizer: str = "llama3"
    family: str = "kafilorn"
    tie_embeddings: bool = False

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @property
    def is_moe(self) -> bool:
        return False            # its experts are not sharded: the engine's expert-parallel wiring does not apply

    @property
    def has_state(self) -> bool:
        return any(L.mixer.kind == "mlstm" for L in self.layers)

    @classmethod
    def from_dict(cls, d: dict, name: str = "kafilorn") -> "KafilornConfig":
        layers = []
        for i, L in enumerate(d["layers"]):
            if L["type"] not in _KAFILORN_MIXERS:
                raise ValueError(f"layer {i}: unknown mixer type {L['type']!r}")
            mixer = _KAFILORN_MIXERS[L["type"]].from_dict(L["mixer"])
            layers.append(KafilornLayer(mixer, FeedForwardSpec.from_dict(L["mlp"]) if L.get("mlp") is not None else None))
        for i, L in enumerate(layers):
            m = L.mixer
            if m.kind == "latent_attention" and m.kv_from >= 0:
                src = layers[m.kv_from].mixer if 0 <= m.kv_from < i else None
                if (src is None or src.kind != "latent_attention" or src.kv_from >= 0 or
                        (src.kv_rank, src.rot_dim, src.rot_dims, src.rot_base) != (m.kv_rank, m.rot_dim, m.rot_dims, m.rot_base)):
                    raise ValueError(f"layer {i}: kv_from {m.kv_from} must name an earlier latent-attention layer with "
                                     "its own key/value latent of the same sizes and rotation")
        emb = d.get("embedding") or {}
        return cls(name=name, vocab_size=int(d["vocab"]), hidden=int(d["width"]), norm_eps=float(d["norm"]["eps"]),
                   streams=int(d.get("streams") or 0), embed_scale=float(emb.get("scale", 1.0)),
                   logit_scale=float(d.get("logit_scale", 1.0)), layers=tuple(layers))

    def to_dict(self) -> dict:
        d = {"architecture": "Kafilorn", "vocab": self.vocab_size, "width": self.hidden, "norm": {"eps": self.norm_eps},
             "embedding": {"scale": self.embed_scale}, "logit_scale": self.logit_scale,
             "layers": [{"type": L.mixer.kind, "mixer": L.mixer.to_dict(), "mlp": L.mlp.to_dict() if L.mlp else None}
                        for L in self.layers]}
        if self.streams:
            d["streams"] = self.streams
        return d

    def num_params(self) -> int:
        h = self.hidden
        n = 2 * self.vocab_size * h + h
        for L in self.layers:
            m, f = L.mixer, L.mlp
            if m.kind == "mlstm":
                n += h * m.heads * (2 * m.dim + 3 * m.vdim + 2) + m.heads * (m.vdim + 2)
            else:
                n += h * m.q_rank + m.q_rank * (1 + m.heads * (m.dim + m.rot_dim)) + m.heads * (m.kv_rank * (m.dim + m.vdim) + m.vdim * h + 1)
                if m.kv_from < 0:
                    n += h * (m.kv_rank + m.rot_dim) + m.kv_rank
            if f is not None:
                n += 2 * h * f.ff if f.kind == "dense" else 3 * h * (f.ff * f.experts + f.shared_ff) + f.experts * (h + 1)
            n += 2 * h + 2 * (2 * self.streams + self.streams ** 2)
        return n

    def default_step_tokens(self) -> int:
        return 8192

    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        """Paged cache per token: the latent and the shared rotated key part of every layer that owns them."""
        return max(1, sum((L.mixer.kv_rank + L.mixer.rot_dim) * dtype_bytes for L in self.layers
                          if L.mixer.kind == "latent_attention" and L.mixer.kv_from < 0))

    def state_bytes_per_slot(self) -> int:
        """Recurrent state per sequence slot (fp32 in every engine dtype)."""
        return sum(L.mixer.state_floats() * 4 for L in self.layers if L.mixer.kind == "mlstm")


def kafilorn_uniform(name: str, blocks: int, hidden: int, heads: int, vocab: int, ff: int, experts: int = 8, top: int = 2,
                     expert_ff: int = 0, window: int = 1024, streams: int = 2, kv_rank: int = 0, q_rank: int = 0,
                     dim: int = 0, rot_dim: int = 0) -> KafilornConfig:
    """`blocks` repetitions of (mLSTM + dense, latent attention + experts, latent attention on the previous layer's
    cache + dense): a regular Kafilorn of given width (benchmarks, tests)."""
    dim = dim or hidden // heads
    rot_dim = rot_dim or dim // 2
    ml = MLSTMSpec(heads, dim, dim, 15.0)
    dense = FeedForwardSpec("dense", ff)
    groups = next(g for g in (4, 3, 2, 1) if experts % g == 0)
    keep = next(k for k in range(max(1, groups // 2), groups + 1) if k * (experts // groups) >= top)
    moe = FeedForwardSpec("moe", expert_ff or ff // 4, experts=experts, top=top, groups=groups, keep_groups=keep,
                          shared_ff=expert_ff or ff // 4)
    layers = []
    for b in range(blocks):
        own = 3 * b + 1
        att = dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=dim, q_rank=q_rank or hidden // 2, kv_rank=kv_rank or hidden // 4,
                   window=window, rot_dims=rot_dim, rot_base=10000.0, scale=(dim + rot_dim) ** -0.5)
        layers += [KafilornLayer(ml, dense), KafilornLayer(LatentAttentionSpec(**att), moe),
                   KafilornLayer(LatentAttentionSpec(**att, kv_from=own), dense)]
    return KafilornConfig(name, vocab, hidden, 1e-6, streams, 1.0, 1.0, tuple(layers))


# ------------------------------------------------------------------------------------------------
# Suvapel: layers listed one by one; one Dynamic-Tanh norm per layer whose output feeds the mixer and the
# feed-forward side by side; a layer's mixer is a gated delta rule (recurrent matrix memory with short
# convolutions, state slots) or that beside sliding-window attention (short convolutions, YaRN-scaled rotary
# positions, kept first tokens, per-head output gate); a gated feed-forward with biases or none; after it a
# per-layer token input from a second embedding table.
@dataclasses.dataclass(frozen=True)
class RotarySpec:
    """Rotary positions on the first `dims` entries of a head, pairs (i, i + dims/2), frequency base^(-2i/dims);
    factor > 0: YaRN scaling (frequencies below the `slow` turn count over `original` positions divided by
    `factor`, above `fast` kept, a linear ramp between; cos and sin scaled by 0.1 ln(factor) + 1)."""
    dims: int = 0
    base: float = 10000.0
    factor: float = 0.0
    original: int = 0
    fast: float = 32.0
    slow: float = 1.0

    @classmethod
    def from_dict(cls, rot: Optional[dict]) -> "RotarySpec":
        if not rot:
            return cls()
        sc = rot.get("scaling")
        if not sc:
            return cls(int(rot["dims"]), float(rot["base"]))
        return cls(int(rot["dims"]), float(rot["base"]), float(sc["factor"]), int(sc["original"]), float(sc["fast"]),
                   float(sc["slow"]))

    def to_dict(self) -> Optional[dict]:
        if not self.dims:
            return None
        d = {"dims": self.dims, "base": self.base}
        if self.factor > 0:
            d["scaling"] = {"factor": self.factor, "original": self.original, "fast": self.fast, "slow": self.slow}
        return d

    def frequencies(self):
        """(frequencies [dims / 2] as float64 list, magnitude factor of cos and sin)."""
        import math

        half = self.dims // 2
        f = [float(self.base) ** (-2.0 * i / self.dims) for i in range(half)]
        if self.factor <= 0 or half == 0:
            return f, 1.0

        def turn_dim(turns: float) -> float:
            return self.dims * math.log(self.original / (2.0 * math.pi * turns)) / (2.0 * math.log(self.base))

        lo = max(math.floor(turn_dim(self.fast)), 0)
        hi = min(math.ceil(turn_dim(self.slow)), self.dims - 1)
        out = []
        for i in range(half):
            ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
            out.append(f[i] / self.factor * ramp + f[i] * (1.0 - ramp))
        return out, 0.1 * math.log(self.factor) + 1.0


@dataclasses.dataclass(frozen=True)
class SlidingAttentionSpec:
    """Softmax attention with grouped keys / values, a short causal convolution on q, k and v, rotary positions,
    a sliding window that also keeps the sequence's first tokens, and a sigmoid gate per head on the output."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int                   # taps of the short convolution (1: none)
    window: int                 # position i sees j <= i with i - j < window (0: all) ...
    keep_first: int             # ... or j < keep_first
    rot: RotarySpec
    scale: float
    kind: str = "sliding_attention"

    @classmethod
    def from_dict(cls, m: dict) -> "SlidingAttentionSpec":
        mask = m.get("mask") or {}
        spec = cls(heads=int(m["heads"]), kv_heads=int(m["kv_heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                   conv=int(m.get("conv") or 1), window=int(mask.get("size") or 0), keep_first=int(mask.get("keep_first") or 0),
                   rot=RotarySpec.from_dict(m.get("rot")), scale=float(m["scale"]))
        if spec.heads % spec.kv_heads or spec.conv < 1 or spec.window < 0 or spec.keep_first < 0:
            raise ValueError(f"bad attention sizes: {spec}")
        if spec.rot.dims % 2 or spec.rot.dims > spec.dim:
            raise ValueError(f"bad rotary dims {spec.rot.dims} for head size {spec.dim}")
        return spec

    def to_dict(self) -> dict:
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "conv": self.conv,
             "scale": self.scale}
        if self.window or self.keep_first:
            d["mask"] = {"size": self.window, "keep_first": self.keep_first}
        if self.rot.dims:
            d["rot"] = self.rot.to_dict()
        return d


@dataclasses.dataclass(frozen=True)
class DeltaSpec:
    """Gated delta rule: per head a [dim, vdim] memory that is decayed, corrected towards the value along the
    unit key, and read with the query; q / k come in kv_heads groups.  channel_decay: one decay per head and key
    channel (through a low-rank pair, with a sigmoid low-rank output gate) instead of one per head (silu gate).
    low_rank: the inner size of those pairs when weights are drawn at random; a checkpoint's tensors give theirs."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    channel_decay: bool = False
    low_rank: int = 16
    kind: str = "delta"

    @classmethod
    def from_dict(cls, m: dict, channel_decay: bool = False) -> "DeltaSpec":
        spec = cls(heads=int(m["heads"]), kv_heads=int(m["kv_heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                   conv=int(m.get("conv") or 1), channel_decay=channel_decay)
        if spec.heads % spec.kv_heads or spec.conv < 1:
            raise ValueError(f"bad delta-rule sizes: {spec}")
        return spec

    def to_dict(self) -> dict:
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "conv": self.conv}

    def state_floats(self) -> int:
        return self.heads * self.dim * self.vdim

    def conv_channels(self) -> int:
        return 2 * self.kv_heads * self.dim + self.heads * self.vdim


@dataclasses.dataclass(frozen=True)
class ParallelMixerSpec:
    """Attention and a delta rule side by side on the same input: left_scale * left + right_scale * right."""
    left: SlidingAttentionSpec
    right: DeltaSpec
    left_scale: float
    right_scale: float
    kind: str = "parallel"

    @classmethod
    def from_dict(cls, m: dict) -> "ParallelMixerSpec":
        return cls(SlidingAttentionSpec.from_dict(m["left"]), DeltaSpec.from_dict(m["right"], channel_decay=True),
                   float(m["left_scale"]), float(m["right_scale"]))

    def to_dict(self) -> dict:
        return {"left": self.left.to_dict(), "right": self.right.to_dict(), "left_scale": self.left_scale,
                "right_scale": self.right_scale}


@dataclasses.dataclass(frozen=True)
class SuvapelLayer:
    mixer: object               # DeltaSpec | ParallelMixerSpec
    ff: int = 0                 # width of the gated feed-forward; 0: none

    @property
    def delta(self) -> DeltaSpec:
        return self.mixer.right if self.mixer.kind == "parallel" else self.mixer

    @property
    def attention(self) -> Optional[SlidingAttentionSpec]:
        return self.mixer.left if self.mixer.kind == "parallel" else None


@dataclasses.dataclass(frozen=True)
class SuvapelConfig:
    name: str
    vocab_size: int
    hidden: int
    norm_eps: float
    residual_mult: float        # every sublayer result enters the residual times this
    side_dim: int               # per-layer slice of the second embedding table; 0: no token input
    layers: Tuple[SuvapelLayer, ...]
    max_position: int = 1 << 20
    tokenizer: str = "llama3"
    family: str = "suvapel"
    tie_embeddings: bool = False
    is_moe: bool = False
    has_state: bool = True

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, d: dict, name: str = "suvapel") -> "SuvapelConfig":
        layers = []
        for i, L in enumerate(d["layers"]):
            if L["type"] == "delta":
                mixer = DeltaSpec.from_dict(L["mixer"])
            elif L["type"] == "parallel":
                mixer = ParallelMixerSpec.from_dict(L["mixer"])
            else:
                raise ValueError(f"layer {i}: unknown mixer type {L['type']!r}")
            mlp = L.get("mlp")
            if mlp is not None and mlp.get("kind") != "dense":
                raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
            layers.append(SuvapelLayer(mixer, int(mlp["ff"]) if mlp is not None else 0))
        side = d.get("token_side") or {}
        return cls(name=name, vocab_size=int(d["vocab"]), hidden=int(d["width"]), norm_eps=float(d["norm"]["eps"]),
                   residual_mult=float(d.get("residual_mult", 1.0)), side_dim=int(side.get("dim") or 0), layers=tuple(layers))

    def to_dict(self) -> dict:
        d = {"architecture": "Suvapel", "vocab": self.vocab_size, "width": self.hidden, "norm": {"eps": self.norm_eps},
             "residual_mult": self.residual_mult,
             "layers": [{"type": L.mixer.kind, "mixer": L.mixer.to_dict(),
                         "mlp": {"kind": "dense", "ff": L.ff} if L.ff else None} for L in self.layers]}
        if self.side_dim:
            d["token_side"] = {"dim": self.side_dim}
        return d

    def num_params(self) -> int:
        h = self.hidden
        n = 2 * self.vocab_size * h + 2 * h + 1 + self.vocab_size * self.side_dim * len(self.layers)
        for L in self.layers:
            m, a = L.delta, L.attention
            n += h * (m.conv_channels() + m.heads) + m.conv_channels() * m.conv + m.heads * m.vdim * h + 2 * m.heads + m.vdim
            if m.channel_decay:
                n += 2 * m.low_rank * h + m.low_rank * m.heads * (m.dim + m.vdim) + m.heads * m.dim
            else:
                n += h * m.heads * (1 + m.vdim)
            if a is not None:
                c = a.heads * a.dim + a.kv_heads * (a.dim + a.vdim)
                n += c * (h + a.conv) + a.heads * h + a.heads * a.vdim * h
            if L.ff:
                n += 3 * h * L.ff + 2 * L.ff + h
            n += 2 * h + 1 + (2 * self.side_dim * h + h if self.side_dim else 0)
        return n

    def default_step_tokens(self) -> int:
        return 8192

    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        """Paged cache per token: keys and values of every attention half."""
        return max(1, sum(L.attention.kv_heads * (L.attention.dim + L.attention.vdim) * dtype_bytes
                          for L in self.layers if L.attention is not None))

    def state_bytes_per_slot(self, dtype_bytes: int = 2) -> int:
        """Per sequence slot: the delta-rule memories (fp32) and the convolutions' last inputs."""
        n = 0
        for L in self.layers:
            m, a = L.delta, L.attention
            n += m.state_floats() * 4 + (m.conv - 1) * m.conv_channels() * dtype_bytes
            if a is not None:
                n += (a.conv - 1) * (a.heads * a.dim + a.kv_heads * (a.dim + a.vdim)) * dtype_bytes
        return n


def suvapel_uniform(name: str, layers: int, hidden: int, heads: int, kv_heads: int, dim: int, ff: int, vocab: int,
                    window: int = 1024, keep_first: int = 4, side_dim: int = 64, conv: int = 4, every: int = 2,
                    low_rank: int = 64) -> SuvapelConfig:
    """A regular Suvapel (benchmarks, tests): every `every`-th layer a plain delta layer, the others attention
    beside a channel-decay delta rule; all heads of size dim."""
    rot = RotarySpec(dim // 2, 10000.0, 8.0, 4096, 32.0, 1.0)
    att = SlidingAttentionSpec(heads, kv_heads, dim, dim, conv, window, keep_first, rot, dim ** -0.5)
    plain = DeltaSpec(heads, kv_heads, dim, dim, conv, False, low_rank)
    par = ParallelMixerSpec(att, DeltaSpec(heads, kv_heads, dim, dim, conv, True, low_rank), 0.5, 0.5)
    ls = tuple(SuvapelLayer(plain if every and i % every == 0 else par, ff) for i in range(layers))
    return SuvapelConfig(name, vocab, hidden, 1e-5, 1.0, side_dim, ls)


# ------------------------------------------------------------------------------------------------
# Zibinex: layers listed one by one, each x += norm(mixer(norm x)) then x += norm(ff(norm x)) with RMS norms whose
# checkpoint weights are offsets from 1; a layer's mixer is latent attention with direct queries, interleaved YaRN-scaled
# rotary positions and a sigmoid gate per head on the output, or sliding-window attention whose weights are
# sigmoids of the score minus a logarithmic distance bias (no softmax); its feed-forward is a clamped gated unit,
# a mixture of experts with a sigmoid router whose weight scales the expert's input, or absent.  A layer may run on
# another layer's weights with a cache of its own.
@dataclasses.dataclass(frozen=True)
class GatedLatentAttentionSpec:
    """Softmax attention over a cached latent [kv_rank] plus one rotated key part [rot_dim] shared by the heads;
    queries are projected directly, head by head [dim unrotated | rot_dim rotated]; rotary pairs are (2i, 2i + 1);
    head h's result is multiplied by sigmoid of one gate logit per token and head."""
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    window: int                 # position i sees j with 0 <= i - j < window (0: all of 0 .. i)
    rot: RotarySpec
    scale: float
    kind: str = "latent_attention"

    @classmethod
    def from_dict(cls, m: dict) -> "GatedLatentAttentionSpec":
        mask = m.get("mask") or {}
        spec = cls(heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=int(m["rot_dim"]), vdim=int(m["vdim"]),
                   kv_rank=int(m["kv_rank"]), window=int(mask.get("size") or 0), rot=RotarySpec.from_dict(m.get("rot")),
                   scale=float(m["scale"]))
        if spec.rot.dims % 2 or spec.rot.dims > spec.rot_dim or spec.window < 0 or min(spec.heads, spec.kv_rank, spec.vdim) < 1:
            raise ValueError(f"bad latent attention sizes: {spec}")
        return spec

    def to_dict(self) -> dict:
        d = {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim, "kv_rank": self.kv_rank,
             "scale": self.scale}
        if self.window:
            d["mask"] = {"size": self.window}
        if self.rot.dims:
            d["rot"] = self.rot.to_dict()
        return d

    def cache_entries(self) -> int:
        return self.kv_rank + self.rot_dim

    def tensor_sizes(self) -> tuple:
        """What fixes the shapes of the mixer's tensors."""
        return (self.kind, self.heads, self.dim, self.rot_dim, self.vdim, self.kv_rank)


@dataclasses.dataclass(frozen=True)
class SigmoidAttentionSpec:
    """Attention with grouped keys / values, biases on q, k, v, a per-head RMS norm of q and k, no rotation, a
    sliding window, and weights sigmoid(score - r1 ln(1 + r2 distance) + pb) that are not normalised over the keys
    (r1, r2, pb: one learned number per head each)."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    window: int                 # position i sees j with 0 <= i - j < window (0: all of 0 .. i)
    scale: float
    kind: str = "attention"

    @classmethod
    def from_dict(cls, m: dict) -> "SigmoidAttentionSpec":
        mask = m.get("mask") or {}
        spec = cls(heads=int(m["heads"]), kv_heads=int(m["kv_heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                   window=int(mask.get("size") or 0), scale=float(m["scale"]))
        if spec.kv_heads < 1 or spec.heads % spec.kv_heads or spec.window < 0 or min(spec.dim, spec.vdim) < 1:
            raise ValueError(f"bad attention sizes: {spec}")
        return spec

    def to_dict(self) -> dict:
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.window:
            d["mask"] = {"size": self.window}
        return d

    def cache_entries(self) -> int:
        return self.kv_heads * (self.dim + self.vdim)

    def tensor_sizes(self) -> tuple:
        """What fixes the shapes of the mixer's tensors."""
        return (self.kind, self.heads, self.kv_heads, self.dim, self.vdim)


@dataclasses.dataclass(frozen=True)
class ClampedFeedForwardSpec:
    """dense: down(g sigmoid(1.702 g) (u + 1)) with g = min(gate h, limit), u = clamp(up h, -limit, limit).
    moe: `experts` gated experts of width ff (silu), the `top` largest sigmoid router scores chosen per token; a
    chosen expert's score multiplies its input, and the results are summed as they are."""
    kind: str                   # "dense" | "moe"
    ff: int
    limit: float = 0.0
    experts: int = 0
    top: int = 0

    GLU_ALPHA = 1.702           # the sigmoid's slope in the dense unit

    @classmethod
    def from_dict(cls, m: dict) -> "ClampedFeedForwardSpec":
        if m["kind"] == "dense":
            return cls("dense", int(m["ff"]), limit=float(m["limit"]))
        if m["kind"] != "moe":
            raise ValueError(f"unknown feed-forward kind {m['kind']!r}")
        spec = cls("moe", int(m["expert"]["ff"]), experts=int(m["router"]["experts"]), top=int(m["router"]["top"]))
        if not 0 < spec.top <= spec.experts:
            raise ValueError(f"bad router: {spec}")
        return spec

    def to_dict(self) -> dict:
        if self.kind == "dense":
            return {"kind": "dense", "ff": self.ff, "limit": self.limit}
        return {"kind": "moe", "expert": {"ff": self.ff}, "router": {"experts": self.experts, "top": self.top}}

    def tensor_sizes(self) -> tuple:
        """What fixes the shapes of the feed-forward's tensors."""
        return (self.kind, self.ff, self.experts)


@dataclasses.dataclass(frozen=True)
class ZibinexLayer:
    mixer: object               # GatedLatentAttentionSpec | SigmoidAttentionSpec
    mlp: Optional[ClampedFeedForwardSpec]
    weights_of: int = -1        # >= 0: no tensors of its own, runs on that layer's; its cache is its own, and so are the
                                # constants of its entry (window, scale, rotation, limit, top)


_ZIBINEX_MIXERS = {"latent_attention": GatedLatentAttentionSpec, "attention": SigmoidAttentionSpec}


@dataclasses.dataclass(frozen=True)
class ZibinexConfig:
    name: str
    vocab_size: int
    hidden: int
    norm_eps: float
    layers: Tuple[ZibinexLayer, ...]
    max_position: int = 1 << 20
    tokenizer: str = "llama3"
    family: str = "zibinex"
    tie_embeddings: bool = True
    is_moe: bool = False        # its experts are not sharded: the engine's expert-parallel wiring does not apply
    has_state: bool = False

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    def owner(self, i: int) -> int:
        """The layer whose tensors layer i runs on."""
        return self.layers[i].weights_of if self.layers[i].weights_of >= 0 else i

    @classmethod
    def from_dict(cls, d: dict, name: str = "zibinex") -> "ZibinexConfig":
        layers = []
        for i, L in enumerate(d["layers"]):
            if L["type"] not in _ZIBINEX_MIXERS:
                raise ValueError(f"layer {i}: unknown mixer type {L['type']!r}")
            wo = L.get("weights_of")
            layers.append(ZibinexLayer(_ZIBINEX_MIXERS[L["type"]].from_dict(L["mixer"]),
                                       ClampedFeedForwardSpec.from_dict(L["mlp"]) if L.get("mlp") is not None else None,
                                       -1 if wo is None else int(wo)))
        for i, L in enumerate(layers):
            if L.weights_of >= 0:
                src = layers[L.weights_of] if L.weights_of < len(layers) and L.weights_of != i else None
                sizes = lambda l: (l.mixer.tensor_sizes(), l.mlp.tensor_sizes() if l.mlp is not None else None)
                if src is None or src.weights_of >= 0 or sizes(src) != sizes(L):
                    raise ValueError(f"layer {i}: weights_of {L.weights_of} must name another layer of the same sizes "
                                     "that has tensors of its own")
        return cls(name=name, vocab_size=int(d["vocab"]), hidden=int(d["width"]), norm_eps=float(d["norm"]["eps"]),
                   layers=tuple(layers))

    def to_dict(self) -> dict:
        out = []
        for L in self.layers:
            e = {"type": L.mixer.kind, "mixer": L.mixer.to_dict(), "mlp": L.mlp.to_dict() if L.mlp else None}
            if L.weights_of >= 0:
                e["weights_of"] = L.weights_of
            out.append(e)
        return {"architecture": "Zibinex", "vocab": self.vocab_size, "width": self.hidden, "norm": {"eps": self.norm_eps},
                "layers": out}

    def num_params(self) -> int:
        h = self.hidden
        n = self.vocab_size * h + h
        for L in self.layers:
            if L.weights_of >= 0:
                continue
            m, f = L.mixer, L.mlp
            if m.kind == "latent_attention":
                n += h * (m.heads * (m.dim + m.rot_dim + 1) + m.kv_rank + m.rot_dim) + m.kv_rank
                n += m.heads * (m.kv_rank * (m.dim + m.vdim) + m.vdim * h)
            else:
                n += (h + 1) * (m.heads * m.dim + m.kv_heads * (m.dim + m.vdim)) + 2 * m.dim + 3 * m.heads + m.heads * m.vdim * h
            n += 2 * h
            if f is not None:
                n += 2 * h + (3 * h * f.ff if f.kind == "dense" else f.experts * (3 * h * f.ff + h))
        return n

    def default_step_tokens(self) -> int:
        return 8192

    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        """Paged cache per token: every layer's own entries, also of a layer that runs on another's weights."""
        return max(1, sum(L.mixer.cache_entries() * dtype_bytes for L in self.layers))


def zibinex_uniform(name: str, layers: int, hidden: int, heads: int, kv_heads: int, dim: int, ff: int, vocab: int,
                    window: int = 1024, kv_rank: int = 0, rot_dim: int = 0, experts: int = 8, top: int = 2,
                    expert_ff: int = 0, share: bool = False, limit: float = 7.0) -> ZibinexConfig:
    """A regular Zibinex (benchmarks, tests): latent attention and sliding sigmoid attention in turn; the first layer
    has the dense feed-forward, the others experts; share: every latent layer after the second layer's runs on its
    weights."""
    rot_dim = rot_dim or dim // 2
    rot = RotarySpec(rot_dim, 10000.0, 8.0, 4096, 32.0, 1.0)
    lat = GatedLatentAttentionSpec(heads, dim, rot_dim, dim, kv_rank or hidden // 4, 0, rot, (dim + rot_dim) ** -0.5)
    att = SigmoidAttentionSpec(heads, kv_heads, dim, dim, window, dim ** -0.5)
    dense = ClampedFeedForwardSpec("dense", ff, limit=limit)
    moe = ClampedFeedForwardSpec("moe", expert_ff or ff // 4, experts=experts, top=top)
    out = []
    for i in range(layers):
        wo = 2 if share and i % 2 == 0 and i > 2 else -1
        out.append(ZibinexLayer(lat if i % 2 == 0 else att, dense if i == 0 else moe, wo))
    return ZibinexConfig(name, vocab, hidden, 1e-6, tuple(out))


# config.json "architecture" -> parser of the file's dict
ARCHITECTURES = {"Vivepel": VivepelConfig.from_dict, "Kafilorn": KafilornConfig.from_dict, "Suvapel": SuvapelConfig.from_dict,
                 "Zibinex": ZibinexConfig.from_dict}


def load_config_dir(path: str):
    """The configuration of a checkpoint folder (config.json + model.safetensors), by its architecture."""
    with open(os.path.join(path, "config.json")) as f:
        d = json.load(f)
    arch = d.get("architecture")
    if arch not in ARCHITECTURES:
        raise ValueError(f"{path}/config.json: unknown architecture {arch!r}; known: {sorted(ARCHITECTURES)}")
    return ARCHITECTURES[arch](d, name=os.path.basename(os.path.normpath(path)) or arch.lower())


PRESETS: Dict[str, ModelConfig] = {
    "llama3-8b": ModelConfig("llama3-8b", "llama", 32, 4096, 32, 8, 128, 14336, 128256, 500000.0),
    "llama3-70b": ModelConfig("llama3-70b", "llama", 80, 8192, 64, 8, 128, 28672, 128256, 500000.0),
    "mixtral-8x7b": ModelConfig("mixtral-8x7b", "mixtral", 32, 4096, 32, 8, 128, 14336, 32000, 1e6,
                                max_position=32768, num_experts=8, top_k=2, tokenizer="llama2"),
    # Same shape family, small enough for CPU tests (fp32 reference) and quick GPU numerics.
    "tiny-llama": ModelConfig("tiny-llama", "llama", 2, 256, 4, 2, 64, 512, 128256, 500000.0),
    "tiny-mixtral": ModelConfig("tiny-mixtral", "mixtral", 2, 256, 4, 2, 64, 384, 32000, 1e6, num_experts=4,
                                top_k=2, tokenizer="llama2"),
    # GPU test model with the real head geometry (head_dim 128, GQA 4) but few layers.
    "llama3-8b-2l": ModelConfig("llama3-8b-2l", "llama", 2, 4096, 32, 8, 128, 14336, 128256, 500000.0),
    # Llama-3-70B geometry (8 KV heads: 1 per rank at TP = 8, GQA group 8) with 2 layers: TP = 4 / 8
    # numerics on one GPU (tests/virtual_tp.py, tests/test_tp_single_gpu.py)
    "llama3-70b-2l": ModelConfig("llama3-70b-2l", "llama", 2, 8192, 64, 8, 128, 28672, 128256, 500000.0),
    # 8 layers of Llama-3-70B: timing a TP group's decode step on one GPU (scripts/bench_tp_persistent_2rank.py)
    "llama3-70b-8l": ModelConfig("llama3-70b-8l", "llama", 8, 8192, 64, 8, 128, 28672, 128256, 500000.0),
    # Llama-3-70B head layout (64 q / 8 kv heads: GQA 8, one KV head per rank at TP = 8) on small
    # layers: CPU multi-process TP = 8 serving tests (gloo), where the 8192-wide layers would not fit
    "llama3-70b-tiny": ModelConfig("llama3-70b-tiny", "llama", 2, 2048, 64, 8, 32, 1024, 128256, 500000.0),
    "mixtral-2l": ModelConfig("mixtral-2l", "mixtral", 2, 4096, 32, 8, 128, 14336, 32000, 1e6, max_position=32768,
                              num_experts=8, top_k=2, tokenizer="llama2"),
    # Vivepel at small sizes (CPU tests) and at the layer sizes of Llama-3-8B (bench.py --arch-compare)
    "tiny-vivepel": vivepel_uniform("tiny-vivepel", 2, 128, 4, 2, 32, 192, 384, chunk=16, rot_dims=12, groups=2),
    "vivepel-8b-2l": vivepel_uniform("vivepel-8b-2l", 2, 4096, 32, 8, 128, 14336, 128256),
    "vivepel-8b": vivepel_uniform("vivepel-8b", 32, 4096, 32, 8, 128, 14336, 128256),
    # Kafilorn at a small size (CPU tests) and at a Llama-3-8B-like width (bench.py --arch-compare)
    "tiny-kafilorn": kafilorn_uniform("tiny-kafilorn", 1, 128, 4, 384, 256, experts=6, top=2, expert_ff=64, window=24,
                                      streams=2, kv_rank=48, q_rank=40, dim=24, rot_dim=8),
    "kafilorn-4k-3l": kafilorn_uniform("kafilorn-4k-3l", 1, 4096, 32, 128256, 14336, experts=8, top=2, expert_ff=3584,
                                       window=1024, streams=2, kv_rank=512, q_rank=1536, dim=128, rot_dim=64),
    # Suvapel at a small size (CPU tests) and at a Llama-3-8B-like width (bench.py --arch-compare)
    "tiny-suvapel": suvapel_uniform("tiny-suvapel", 3, 128, 4, 2, 32, 192, 384, window=24, keep_first=3, side_dim=16,
                                    conv=3, every=3, low_rank=8),
    "suvapel-4k-2l": suvapel_uniform("suvapel-4k-2l", 2, 4096, 32, 8, 128, 14336, 128256),
    # Zibinex at a small size (CPU tests) and at a Llama-3-8B-like width (bench.py --arch-compare)
    "tiny-zibinex": zibinex_uniform("tiny-zibinex", 5, 128, 4, 2, 24, 256, 384, window=20, kv_rank=40, rot_dim=8,
                                    experts=6, top=2, expert_ff=64, share=True, limit=1.25),
    "zibinex-4k-2l": zibinex_uniform("zibinex-4k-2l", 2, 4096, 32, 8, 128, 14336, 128256, kv_rank=512, rot_dim=64,
                                     expert_ff=3584),
}


def get_config(name: str):
    """A preset by name, or a checkpoint folder (its config.json names the architecture)."""
    if name in PRESETS:
        return PRESETS[name]
    if os.path.isdir(name) and os.path.exists(os.path.join(name, "config.json")):
        return load_config_dir(name)
    raise ValueError(f"unknown MODEL {name!r}; choose from {sorted(PRESETS)} or give a checkpoint folder")
