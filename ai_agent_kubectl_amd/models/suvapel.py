"""Suvapel decoder over the engine ops (`ops/mixers.py`).

The residual x [T, W] is fp32.  A layer has one Dynamic-Tanh norm whose output h feeds the mixer and the
feed-forward side by side, then a token input from a second embedding table:
  h = tanh(alpha x) w + b                                       dyt_norm / fused into the update before it
  x <- x + m (mixer(h) + ff(h))                                 residual_mix (fp32 sum of the sublayers' results)
  x <- x + m rms_norm(P (gelu_tanh(G x) * e_layer[token]))      gelu_gate_embed, rms_residual (+ the next layer's h)
Every projection that reads h is one row block of `w_in` (one vendor GEMM per layer, `weights.suvapel_columns`).

Mixers (activations in the engine dtype, bf16 or fp32; what is marked fp32 is fp32 in both):
  delta rule        q | k | v through a short causal convolution + silu over the sequence's conv state
                    (short_conv); unit q, k per head, beta, decay in fp32 (delta_prep); the recurrence over the
                    step's rows from / into the sequence's state slot, fp32 (delta_scan); per-head RMS division,
                    weight and output gate (headnorm_gate: silu gate, or sigmoid of a low-rank pair); output GEMM.
                    The decay is per head, or (beside attention) per head and key channel through a low-rank pair.
  sliding attention q | k | v through a short convolution (no activation); YaRN-scaled rotary positions on q and k,
                    k and v appended to the paged cache (rope_append); softmax attention over the last `window`
                    positions and the first `keep_first`, times a sigmoid gate per head (sliding_attention);
                    output GEMM.
  parallel          left_scale * attention + right_scale * delta rule, both on h.
Feed-forward: down(silu(gate h + b) * (up h + b)) + b.

Cache: per attention layer K [NB, G, BS, D] and V [NB, G, Dv, BS] (a page's values of one entry contiguous) under the engine's single block table.  State:
per layer and state slot the delta-rule memory [H, Dv, D] fp32 and the convolutions' last taps - 1 inputs (engine
dtype), indexed by the sequence's state slot (`AttnMeta.state_slots`); a row at position 0 starts from zeros, so
slots are reused without clearing.  Prefill, chunked prefill, mixed and decode steps all run this forward; the
decode step is shape-static and capturable.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch
import torch.nn.functional as F

from .. import ops
from ..ops import mixers
from .config import SuvapelConfig
from .llama import AttnMeta
from .weights import suvapel_columns


class SuvapelModel:
    supports_block_copy = False     # no sub-block KV copies (ops.kv_block_copy assumes Llama's cache layout)
    supports_prefix_cache = False   # a recurrent state cannot be rebuilt from cached pages

    def __init__(self, cfg: SuvapelConfig, weights: Dict[str, torch.Tensor], comm=None, tp_rank: int = 0,
                 tp_size: int = 1, ep_rank: int = 0, ep_size: int = 1):
        if tp_size != 1 or ep_size != 1:
            raise ValueError("Suvapel runs at TP = 1")
        self.cfg = cfg
        self.W = weights
        self.comm = comm
        self.tp_rank, self.tp_size = 0, 1
        self.device = weights["embed"].device
        self.dtype = weights["embed"].dtype
        self.vocab_offset = 0
        self.layers: List[dict] = []
        self.cols: List[Dict[str, int]] = []
        for i, spec in enumerate(cfg.layers):
            p = f"layers.{i}."
            L = {k[len(p):]: v for k, v in weights.items() if k.startswith(p)}
            L["dyt"] = (L["norm_alpha"], L["norm_w"], L["norm_b"])
            if spec.attention is not None:
                L["rot_mag"] = spec.attention.rot.frequencies()[1]   # YaRN's factor on cos and sin (1 without scaling)
            self.layers.append(L)
            ra = L["w_a2"].shape[1] if "w_a2" in L else 0
            rg = L["w_g2"].shape[1] if "w_g2" in L else 0
            self.cols.append(suvapel_columns(spec, ra, rg))
        self.final_dyt = (weights["norm_alpha"], weights["norm_w"], weights["norm_b"])
        # per layer: (delta-rule memory, its conv state, the attention's conv state)
        self.state: List[Optional[tuple]] = [None] * cfg.num_layers
        # the runner's hooks shared with LlamaModel
        self.persistent = False
        self.mark_layer = -1
        self.mark_event = None
        self.fuse_decode_rope = False
        # debugging / tests: called with (layer index, the residual [T, W] fp32) after every layer
        self.layer_hook = None

    # ---- the runner's model interface ----------------------------------------------------------
    def alloc_cache(self, num_blocks: int, block_size: int):
        """(k_cache, v_cache): per layer [NB, G, BS, D] / [NB, G, Dv, BS] for its attention half (None without one)."""
        ks: List[Optional[torch.Tensor]] = []
        vs: List[Optional[torch.Tensor]] = []
        for L in self.cfg.layers:
            a = L.attention
            if a is None:
                ks.append(None)
                vs.append(None)
            else:
                z = dict(dtype=self.dtype, device=self.device)
                ks.append(torch.zeros((num_blocks, a.kv_heads, block_size, a.dim), **z))
                vs.append(torch.zeros((num_blocks, a.kv_heads, a.vdim, block_size), **z))
        return ks, vs

    def alloc_state(self, num_slots: int) -> None:
        """Recurrent state for `num_slots` live sequences: the memories in fp32, the conv inputs in the engine dtype."""
        for i, L in enumerate(self.cfg.layers):
            m, a = L.delta, L.attention
            S = torch.zeros((num_slots, m.heads, m.vdim, m.dim), dtype=torch.float32, device=self.device)
            cs = (torch.zeros((num_slots, m.conv - 1, m.conv_channels()), dtype=self.dtype, device=self.device)
                  if m.conv > 1 else None)
            acs = None
            if a is not None and a.conv > 1:
                acs = torch.zeros((num_slots, a.conv - 1, a.heads * a.dim + a.kv_heads * (a.dim + a.vdim)),
                                  dtype=self.dtype, device=self.device)
            self.state[i] = (S, cs, acs)

    def persistent_ok(self, B: int = 1) -> bool:
        return False

    def persistent_err_word(self):
        return None

    def persistent_err(self) -> int:
        return 0

    # ---- sublayers -----------------------------------------------------------------------------
    def _delta(self, proj, L, m, col, li, meta: AttnMeta):
        S, cs, _ = self.state[li]
        qs = None if meta.is_decode else meta.q_starts
        GD = m.kv_heads * m.dim
        cv = mixers.short_conv(proj, col["q"], m.conv_channels(), L["conv"], cs, meta.state_slots, qs, meta.positions, True)
        if m.channel_decay:
            a_src, a_off = F.linear(proj[:, col["a"]:col["a"] + L["w_a2"].shape[1]], L["w_a2"]), 0
            g_src, g_off = F.linear(proj[:, col["g"]:col["g"] + L["w_g2"].shape[1]], L["w_g2"]), 0
        else:
            a_src, a_off, g_src, g_off = proj, col["a"], proj, col["g"]
        qk, beta, decay = mixers.delta_prep(cv, proj, col["beta"], a_src, a_off, L["A_log"], L["dt_bias"], m.heads,
                                            m.kv_heads, m.dim, m.channel_decay)
        o = mixers.delta_scan(qk, cv, 2 * GD, beta, decay, S, meta.state_slots, qs, meta.positions, m.heads, m.kv_heads,
                              m.dim, m.vdim)
        o = mixers.headnorm_gate(o, g_src, g_off, L["hnorm"], m.heads, m.vdim, self.cfg.norm_eps, self.dtype,
                                 silu=not m.channel_decay)
        return F.linear(o, L["wo"])

    def _attention(self, proj, L, a, col, li, k_cache, v_cache, meta: AttnMeta):
        qs = None if meta.is_decode else meta.q_starts
        C = a.heads * a.dim + a.kv_heads * (a.dim + a.vdim)
        cv = mixers.short_conv(proj, col["att_q"], C, L["att_conv"], self.state[li][2], meta.state_slots, qs,
                               meta.positions, False)
        q = mixers.rope_append(cv, L.get("inv_freq"), L["rot_mag"], meta.positions, meta.slot_mapping, k_cache, v_cache,
                               a.heads, a.kv_heads, a.dim, a.vdim, a.rot.dims)
        o = mixers.sliding_attention(q, k_cache, v_cache, meta.block_tables, qs, meta.positions, meta.slot_mapping, proj,
                                     col["att_g"], a.window, a.keep_first, a.scale, meta.max_q_len, meta.num_decode)
        return F.linear(o, L["att_wo"])

    # ---- forward -------------------------------------------------------------------------------
    def hidden_states(self, input_ids: torch.Tensor, meta: AttnMeta, k_cache, v_cache) -> torch.Tensor:
        """(the residual after the last layer [T, W] fp32, its final norm [T, W] in the engine dtype)."""
        cfg, eps, mult = self.cfg, self.cfg.norm_eps, self.cfg.residual_mult
        if meta.state_slots is None or (self.layers and self.state[0] is None):
            raise RuntimeError("Suvapel without state slots: the runner must call alloc_state and pass state_slots")
        x = mixers.embed_f32(input_ids, self.W["embed"])
        last = len(self.layers) - 1
        h = mixers.dyt_norm(x, *(self.layers[0]["dyt"] if self.layers else self.final_dyt), self.dtype)
        for li, (L, spec) in enumerate(zip(self.layers, cfg.layers)):
            if li == self.mark_layer and x.is_cuda:   # progress marker (engine lookahead timing)
                self.mark_event = torch.cuda.Event()
                self.mark_event.record()
            col = self.cols[li]
            proj = F.linear(h, L["w_in"])
            ys, cs = [self._delta(proj, L, spec.delta, col, li, meta)], [mult]
            if spec.attention is not None:
                ys.append(self._attention(proj, L, spec.attention, col, li, k_cache[li], v_cache[li], meta))
                cs = [mult * spec.mixer.right_scale, mult * spec.mixer.left_scale]
            if spec.ff:
                ys.append(F.linear(mixers.silu_mul_bias(proj, col["ff"], spec.ff, L["b_gu"]), L["w_down"], L["b_down"]))
                cs.append(mult)
            nxt = self.layers[li + 1]["dyt"] if li < last else self.final_dyt
            if cfg.side_dim:
                xa, _ = mixers.residual_mix(x, ys, cs, self.dtype, want_copy=True)
                g = mixers.gelu_gate_embed(F.linear(xa, L["side_gate"]), self.W["side_embed"], input_ids, li * cfg.side_dim)
                h = mixers.rms_residual(x, F.linear(g, L["side_proj"]), L["side_norm"], mult, eps, self.dtype, nxt)
            else:
                _, h = mixers.residual_mix(x, ys, cs, self.dtype, dyt=nxt)
            if self.layer_hook is not None:
                self.layer_hook(li, x)
        return x, h

    def forward(self, input_ids: torch.Tensor, meta: AttnMeta, k_cache, v_cache) -> torch.Tensor:
        """The final-normed hidden state of the rows `meta.logits_indices`: [S, W] in the engine dtype."""
        _, h = self.hidden_states(input_ids, meta, k_cache, v_cache)
        if not (meta.is_decode and meta.logits_indices.shape[0] == h.shape[0]):
            h = h.index_select(0, meta.logits_indices)
        return h

    def logits(self, hidden_last: torch.Tensor) -> torch.Tensor:
        return F.linear(hidden_last, self.W["lm_head"])

    def sample(self, hidden_last: torch.Tensor, mask_bits: Optional[torch.Tensor],
               mask_idx: Optional[torch.Tensor]) -> torch.Tensor:
        """Greedy next tokens under the SAFE_DECODE mask: [S] int32."""
        logits = F.linear(hidden_last, self.W["lm_head"])
        if logits.dtype == torch.bfloat16 and logits.shape[1] % 8 == 0 and logits.is_cuda:
            return ops.masked_argmax(logits, mask_bits, mask_idx)[0]
        return ops.ref.masked_argmax(logits, mask_bits, mask_idx)[0]
