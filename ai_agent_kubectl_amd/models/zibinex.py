"""Zibinex decoder over the engine ops (`ops/mixers.py`).

The residual x [T, W] is fp32.  A layer is x += n1b(mixer(n1(x))), then (if it has one) x += n2b(ff(n2(x))), every
n an RMS norm x / sqrt(mean(x^2) + eps) * (1 + w), w being what the checkpoint holds (the loader keeps 1 + w in fp32):
  h = norm(x)                                   group_rmsnorm with one group / fused into the update before it
  x += norm(y); h = next norm(x)                post_norm_residual (no layer scale)

Mixers (activations in the engine dtype, bf16 or fp32; what is marked fp32 is fp32 in both):
  latent attention  [c | k_r | q | g] = h @ w_in^T (one GEMM); RMS norm of c and rotary on k_r appended to the paged
                    cache (latent_prep without a query latent); rotary on q's rotated parts, the unrotated parts
                    carried into the latent space by a batched GEMM with w_uk (rope_split_q, bmm); causal softmax
                    attention over the cached rows with the latent as the value (window_attention, no sink); w_uv by
                    a batched GEMM; head h times sigmoid(g_h) while the heads are laid side by side (head_gate);
                    output GEMM.  Rotary pairs are (2i, 2i + 1); the frequencies and the magnitude of cos and sin
                    carry the YaRN scaling (`RotarySpec.frequencies`).
  attention         [q | k | v] = h @ w_qkv^T + b (one GEMM); per-head RMS norm of q and k (plain weights), k and v
                    appended to the paged cache (rope_append without rotation); sliding-window attention whose
                    weights are sigmoid(score - r1 ln(1 + r2 distance) + pb), not normalised (sliding_attention with
                    `dist`); output GEMM.
Feed-forwards: dense down(g sigmoid(1.702 g) (u + 1)), g = min(gate h, limit), u = clamp(up h, +-limit) (glu_clamp);
or experts chosen by a sigmoid router (moe_route: sigmoid scores, no renormalisation) whose score multiplies the
expert's input, summed in fp32 (moe_experts with scale_input).

A layer with `weights_of` runs on its owner's tensors (the same dict) with a cache of its own and the constants of
its own entry (window, scale, rotary table, limit, top).  Cache: per layer
either the latent rows [NB, BS, kv_rank + rot_dim] or K [NB, G, BS, D] and V [NB, G, Dv, BS], under the engine's single
block table.  No recurrent state.  Prefill, chunked prefill, mixed and decode steps all run this forward; the decode
step is shape-static and capturable.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch
import torch.nn.functional as F

from .. import ops
from ..ops import mixers
from .config import ZibinexConfig
from .llama import AttnMeta
from .weights import zibinex_columns


class ZibinexModel:
    supports_block_copy = False     # no sub-block KV copies (ops.kv_block_copy assumes Llama's cache layout)

    def __init__(self, cfg: ZibinexConfig, weights: Dict[str, torch.Tensor], comm=None, tp_rank: int = 0,
                 tp_size: int = 1, ep_rank: int = 0, ep_size: int = 1):
        if tp_size != 1 or ep_size != 1:
            raise ValueError("Zibinex runs at TP = 1")
        self.cfg = cfg
        self.W = weights
        self.comm = comm
        self.tp_rank, self.tp_size = 0, 1
        self.device = weights["embed"].device
        self.dtype = weights["embed"].dtype
        self.vocab_offset = 0
        own: Dict[int, dict] = {}
        for i, spec in enumerate(cfg.layers):
            if spec.weights_of < 0:
                p = f"layers.{i}."
                own[i] = {k[len(p):]: v for k, v in weights.items() if k.startswith(p)}
        self.layers: List[dict] = [own[cfg.owner(i)] for i in range(cfg.num_layers)]
        # per layer, from its own entry: the rotary table (frequencies in float64 rounded once to fp32; the angle is
        # position * frequency in fp32), YaRN's factor on cos and sin (1 without scaling), the fused row's columns
        self.rotary: List[Optional[tuple]] = [None] * cfg.num_layers
        for i, spec in enumerate(cfg.layers):
            if spec.mixer.kind == "latent_attention":
                f, mag = spec.mixer.rot.frequencies()
                inv = torch.tensor(f, dtype=torch.float64).to(device=self.device, dtype=torch.float32)
                self.rotary[i] = (inv, mag, zibinex_columns(spec.mixer))
        # the runner's hooks shared with LlamaModel
        self.persistent = False
        self.mark_layer = -1
        self.mark_event = None
        self.fuse_decode_rope = False
        # debugging / tests: called with (layer index, the residual [T, W] fp32) after every layer
        self.layer_hook = None

    # ---- the runner's model interface ----------------------------------------------------------
    def alloc_cache(self, num_blocks: int, block_size: int):
        """(k_cache, v_cache) per layer: latent rows [NB, BS, kv_rank + rot_dim] (no value tensor), or keys
        [NB, G, BS, D] and values [NB, G, Dv, BS]; zero-filled; every layer has its own, whoever owns its weights."""
        ks: List[torch.Tensor] = []
        vs: List[Optional[torch.Tensor]] = []
        z = dict(dtype=self.dtype, device=self.device)
        for L in self.cfg.layers:
            m = L.mixer
            if m.kind == "latent_attention":
                ks.append(torch.zeros((num_blocks, block_size, m.kv_rank + m.rot_dim), **z))
                vs.append(None)
            else:
                ks.append(torch.zeros((num_blocks, m.kv_heads, block_size, m.dim), **z))
                vs.append(torch.zeros((num_blocks, m.kv_heads, m.vdim, block_size), **z))
        return ks, vs

    def persistent_ok(self, B: int = 1) -> bool:
        return False

    def persistent_err_word(self):
        return None

    def persistent_err(self) -> int:
        return 0

    # ---- sublayers -----------------------------------------------------------------------------
    def _latent_attention(self, h, L, m, li, cache, meta: AttnMeta):
        (inv_freq, mag, col), eps = self.rotary[li], self.cfg.norm_eps
        proj = F.linear(h, L["w_in"])                                  # [T, c | k_r | q | g]
        mixers.latent_prep(proj, 0, m.kv_rank, m.rot_dim, None, L["kv_norm"], inv_freq, meta.positions,
                           meta.slot_mapping, cache, m.rot.dims, eps, interleaved=True, mag=mag)
        qn, qr = mixers.rope_split_q(proj, inv_freq, meta.positions, m.heads, m.dim, m.rot_dim, m.rot.dims,
                                     interleaved=True, mag=mag, off=col["q"])
        q_lat = torch.bmm(qn, L["w_uk"])                               # [H, T, R]
        o_lat = mixers.window_attention(q_lat, qr, cache, meta.block_tables, None if meta.is_decode else meta.q_starts,
                                        meta.positions, meta.slot_mapping, None, m.window, m.scale)
        o = torch.bmm(o_lat, L["w_uv"].transpose(1, 2))                # [H, T, Dv]
        return F.linear(mixers.head_gate(o, proj, col["g"]), L["wo"])

    def _attention(self, h, L, m, k_cache, v_cache, meta: AttnMeta):
        qkv = F.linear(h, L["w_qkv"], L["b_qkv"])
        q = mixers.rope_append(qkv, None, 1.0, meta.positions, meta.slot_mapping, k_cache, v_cache, m.heads, m.kv_heads,
                               m.dim, m.vdim, 0, L["q_norm"], L["k_norm"], self.cfg.norm_eps)
        o = mixers.sliding_attention(q, k_cache, v_cache, meta.block_tables, None if meta.is_decode else meta.q_starts,
                                     meta.positions, meta.slot_mapping, None, 0, m.window, 0, m.scale, meta.max_q_len,
                                     meta.num_decode, dist=L["dist"])
        return F.linear(o, L["wo"])

    def _feed_forward(self, h, L, f):
        if f.kind == "dense":
            return F.linear(mixers.glu_clamp(F.linear(h, L["w_gu"]), f.limit, f.GLU_ALPHA), L["w_down"])
        ids, w = mixers.moe_route(h, L["w_router"], None, f.top, 1, 1, sigmoid=True, renorm=False)
        return mixers.moe_experts(h, L["w_gu_e"], L["w_dn_e"], ids, w, scale_input=True)      # fp32

    # ---- forward -------------------------------------------------------------------------------
    def hidden_states(self, input_ids: torch.Tensor, meta: AttnMeta, k_cache, v_cache) -> torch.Tensor:
        """The residual after the last layer for every row: [T, W] fp32."""
        cfg, eps = self.cfg, self.cfg.norm_eps
        x = mixers.embed_f32(input_ids, self.W["embed"])
        last = len(self.layers) - 1
        h = mixers.group_rmsnorm(x, self.layers[0]["norm1"], 1, eps, out_dtype=self.dtype) if self.layers else None
        for li, (L, spec) in enumerate(zip(self.layers, cfg.layers)):
            if li == self.mark_layer and x.is_cuda:   # progress marker (engine lookahead timing)
                self.mark_event = torch.cuda.Event()
                self.mark_event.record()
            m, f = spec.mixer, spec.mlp
            if m.kind == "latent_attention":
                y = self._latent_attention(h, L, m, li, k_cache[li], meta)
            else:
                y = self._attention(h, L, m, k_cache[li], v_cache[li], meta)
            nxt = self.layers[li + 1]["norm1"] if li < last else None
            if f is not None:
                h = mixers.post_norm_residual(x, y, L["norm1b"], None, L["norm2"], 1, eps)
                h = mixers.post_norm_residual(x, self._feed_forward(h, L, f), L["norm2b"], None, nxt, 1, eps, self.dtype)
            else:
                h = mixers.post_norm_residual(x, y, L["norm1b"], None, nxt, 1, eps)
            if self.layer_hook is not None:
                self.layer_hook(li, x)
        return x

    def forward(self, input_ids: torch.Tensor, meta: AttnMeta, k_cache, v_cache) -> torch.Tensor:
        """The final-normed hidden state of the rows `meta.logits_indices`: [S, W] in the engine dtype."""
        x = self.hidden_states(input_ids, meta, k_cache, v_cache)
        if not (meta.is_decode and meta.logits_indices.shape[0] == x.shape[0]):
            x = x.index_select(0, meta.logits_indices)
        return mixers.group_rmsnorm(x, self.W["norm"], 1, self.cfg.norm_eps, out_dtype=self.dtype)

    def logits(self, hidden_last: torch.Tensor) -> torch.Tensor:
        return F.linear(hidden_last, self.W["lm_head"])

    def sample(self, hidden_last: torch.Tensor, mask_bits: Optional[torch.Tensor],
               mask_idx: Optional[torch.Tensor]) -> torch.Tensor:
        """Greedy next tokens under the SAFE_DECODE mask: [S] int32."""
        logits = self.logits(hidden_last)
        if logits.dtype == torch.bfloat16 and logits.shape[1] % 8 == 0 and logits.is_cuda:
            return ops.masked_argmax(logits, mask_bits, mask_idx)[0]
        return ops.ref.masked_argmax(logits, mask_bits, mask_idx)[0]
