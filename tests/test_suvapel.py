"""Suvapel in the engine against the plain oracle (tests/suvapel_oracle.py).

Every test makes its own small configuration and random (or crafted) weights, writes them as a checkpoint
folder (config.json + model.safetensors: the reader and the loader are under test too), builds the engine on it
and compares logits with the oracle's whole-sequence forward.  The same bodies run on the CPU (the ops' torch
references) and, marked `gpu`, on the HIP kernels in fp32 and bf16.
"""
import json
import os

import numpy as np
import pytest
import torch

import suvapel_oracle as oracle
from suvapel_oracle import attention_cfg, delta_layer, delta_mixer_cfg, make_config, parallel_layer

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
BS = 16


def write_checkpoint(path, config, W):
    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(config, f)
    save_file({k: v.contiguous() for k, v in W.items()}, os.path.join(path, "model.safetensors"))
    return str(path)


def session(path, device, dtype="float32", max_tokens=256, max_requests=4):
    from ai_agent_kubectl_amd.engine.trace import TraceSession

    return TraceSession(path, dtype=dtype, max_tokens=max_tokens, device=device, max_requests=max_requests)


def replay(sess, tokens, cuts, rid="r", end=True):
    """Feed `tokens` in portions of the sizes `cuts`; logits of every position [n, vocab]."""
    out, at = [], 0
    for c in cuts:
        part = tokens[at:at + c]
        last = at + c >= len(tokens)
        out.append(sess.step([{"id": rid, "tokens": part, "want": list(range(len(part)))}], [rid] if last and end else []))
        at += c
    assert at == len(tokens)
    return np.concatenate(out)


def rel_err(got, want):
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    w = want - want.mean(-1, keepdims=True)
    return float(np.sqrt((d ** 2).mean(-1)).max() / np.sqrt((w ** 2).mean()))


def tol(dtype):
    return 2e-4 if dtype == "float32" else 6e-2


def tokens_for(config, n, seed=0):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, config["vocab"], (n,), generator=g).tolist()


def want_logits(config, W, tokens, layer_out=None):
    return oracle.forward(config, oracle.as_arrays(W), tokens, layer_out)


def variant(name):
    if name == "base":           # both kinds of layer; window 8 is half a page; taps 4, 2 and 3
        return make_config([delta_layer(), parallel_layer(), parallel_layer(ff=0), delta_layer(heads=4, kv_heads=4, dim=4, vdim=6, conv=2)])
    if name == "attention_first":  # odd sizes: heads of 10 / 7 entries, one key/value head, window 21 over a page border,
        # rotation on the whole head without scaling, five taps, no token input, multiplier 1
        return make_config([parallel_layer(left=attention_cfg(heads=3, kv_heads=1, dim=10, vdim=7, conv=5, window=21, keep_first=5,
                                                              rot_dims=10, scaling=None),
                                           right=delta_mixer_cfg(heads=3, kv_heads=3, dim=5, vdim=9, conv=1), left_scale=1.0,
                                           right_scale=0.25, ff=33),
                            delta_layer(heads=3, kv_heads=1, dim=6, vdim=10, conv=5, ff=0)],
                           width=36, vocab=80, side=0, mult=1.0)
    if name == "no_window":      # no mask (all earlier keys), no rotation, one tap (no convolution), one head
        return make_config([parallel_layer(left=attention_cfg(heads=1, kv_heads=1, dim=8, vdim=8, conv=1, window=0, rot_dims=0),
                                           right=delta_mixer_cfg(heads=1, kv_heads=1, dim=16, vdim=4, conv=2)),
                            parallel_layer(left=attention_cfg(heads=2, kv_heads=2, dim=12, vdim=20, conv=2, window=1, keep_first=0,
                                                              rot_dims=4, scaling=(16.0, 32, 4.0, 0.5)), ff=16)],
                           width=24, vocab=72, side=3, mult=0.5)
    if name == "keep_all":       # more kept first tokens than the window holds; the kept span meets the window
        return make_config([parallel_layer(left=attention_cfg(window=3, keep_first=9)), delta_layer(ff=8)], width=16, vocab=64, side=1)
    raise KeyError(name)


VARIANTS = ["base", "attention_first", "no_window", "keep_all"]


def model_for(tmp_path, name, seed=0):
    c = variant(name)
    W = oracle.random_tensors(c, seed)
    return c, W, write_checkpoint(tmp_path / name, c, W)


def close(got, want, rtol=1e-4, atol=1e-4):
    return np.allclose(np.asarray(got.detach().cpu().double()), np.asarray(want), rtol=rtol, atol=atol)


# ---------------------------------------------------------------------------------------------------
# each mechanism alone: ops.mixers (torch reference on CPU, HIP kernel on GPU) against the oracle
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("width", [24, 100, 513])
def test_dyt_norm_and_residual_rows(device, width):
    from ai_agent_kubectl_amd.ops import mixers

    g = torch.Generator().manual_seed(width)
    x = torch.randn(5, width, generator=g) * 3 + 1
    ys = [torch.randn(5, width, generator=g) for _ in range(3)]
    alpha, w, b = torch.tensor([0.6]), torch.rand(width, generator=g) + 0.5, torch.randn(width, generator=g)
    dy = (alpha.to(device), w.to(device), b.to(device))
    want_h = oracle.dyt(x.double().numpy(), 0.6, w.double().numpy(), b.double().numpy())
    assert close(mixers.dyt_norm(x.to(device), *dy, torch.float32), want_h)
    assert not np.allclose(oracle.rms_div(x.double().numpy(), 1e-5) * w.double().numpy(), want_h, atol=1e-2)   # no statistics in it
    for n in (1, 2, 3):
        coefs = [0.65, -0.3, 1.25][:n]
        new = x.double() + sum(c * y.double() for c, y in zip(coefs, ys))
        xd = x.clone().to(device)
        xa, h = mixers.residual_mix(xd, [y.to(device) for y in ys[:n]], coefs, torch.float32, want_copy=True, dyt=dy)
        assert close(xd, new, 1e-5, 1e-5) and close(xa, new, 1e-5, 1e-5)
        assert close(h, oracle.dyt(new.numpy(), 0.6, w.double().numpy(), b.double().numpy()))
        xd = x.clone().to(device)
        assert mixers.residual_mix(xd, [y.to(device) for y in ys[:n]], coefs, torch.float32) == (None, None) and close(xd, new, 1e-5, 1e-5)
    wn = torch.rand(width, generator=g)
    y = ys[0] * 5 + 2
    new = x.double().numpy() + 0.65 * oracle.rms_div(y.double().numpy(), 1e-5) * wn.double().numpy()
    for with_dyt in (False, True):
        xd = x.clone().to(device)
        h = mixers.rms_residual(xd, y.to(device), wn.to(device), 0.65, 1e-5, torch.float32, dy if with_dyt else None)
        assert close(xd, new, 1e-5, 1e-5)
        assert (h is None) if not with_dyt else close(h, oracle.dyt(new, 0.6, w.double().numpy(), b.double().numpy()))


@pytest.mark.parametrize("device", DEVICES)
def test_token_gate_and_gated_ff_rows(device):
    from ai_agent_kubectl_amd.ops import mixers

    g = torch.Generator().manual_seed(3)
    z, table = torch.randn(6, 7, generator=g) * 2, torch.randn(20, 35, generator=g)
    ids = torch.tensor([3, 0, 19, 7, 7, 11], dtype=torch.int32)
    got = mixers.gelu_gate_embed(z.to(device), table.to(device), ids.to(device), 14)
    assert close(got, oracle.gelu_tanh(z.double().numpy()) * table.double().numpy()[ids.long().numpy(), 14:21])
    proj, bias = torch.randn(6, 64, generator=g), torch.randn(2 * 13, generator=g)
    got = mixers.silu_mul_bias(proj.to(device), 8, 13, bias.to(device))
    p, bb = proj.double().numpy(), bias.double().numpy()
    assert close(got, oracle.silu(p[:, 8:21] + bb[:13]) * (p[:, 21:34] + bb[13:]))
    # head norm with a silu gate next to the sigmoid one
    o, gate, w = torch.randn(6, 3 * 10, generator=g) * 4, torch.randn(6, 40, generator=g), torch.rand(30, generator=g) + 0.5
    normed = oracle.rms_div(o.double().numpy().reshape(6, 3, 10), 1e-5).reshape(6, 30) * w.double().numpy()
    gg = gate.double().numpy()[:, 5:35]
    for silu, fn in ((True, oracle.silu), (False, oracle.sigmoid)):
        got = mixers.headnorm_gate(o.to(device), gate.to(device), 5, w.to(device), 3, 10, 1e-5, torch.float32, silu=silu)
        assert close(got, normed * fn(gg))


def _seq_meta(lens, device):
    """q_starts for rows laid out sequence after sequence."""
    return torch.tensor(np.concatenate([[0], np.cumsum(lens)]), dtype=torch.int32, device=device)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("taps,C,act", [(1, 5, True), (2, 7, False), (3, 300, True), (4, 64, False), (8, 9, True)])
def test_short_conv_whole_portions_and_decode(device, taps, C, act):
    """One sequence of 23 rows: whole, in portions (down to one row, shorter than the taps), and row by row through
    the decode form, each from a slot that still holds another sequence's inputs."""
    from ai_agent_kubectl_amd.ops import mixers

    g = torch.Generator().manual_seed(taps)
    n, off = 23, 3
    proj = torch.randn(n, C + 11, generator=g)
    w = torch.randn(C, taps, generator=g)
    y = oracle.short_conv(proj.double().numpy()[:, off:off + C], w.double().numpy())
    want = oracle.silu(y) if act else y
    for cuts in ([n], [1, 2, 1, 5, 1, 1, 9, 3], [2] * 11 + [1]):
        state = torch.randn(3, taps - 1, C, generator=g).to(device) * 50 if taps > 1 else None   # stale values
        got, at = [], 0
        for c in cuts:
            pos = torch.arange(at, at + c, dtype=torch.int32, device=device)
            got.append(mixers.short_conv(proj[at:at + c].contiguous().to(device), off, C, w.t().contiguous().to(device), state,
                                         torch.tensor([1], dtype=torch.int32, device=device), _seq_meta([c], device), pos, act))
            at += c
        assert close(torch.cat(got), want)
    # decode form: three sequences at different positions in one step, row t is sequence t; slot -1 is a padding row
    state = torch.zeros(4, taps - 1, C).to(device) if taps > 1 else None
    outs = []
    for t in range(n):
        rows = torch.stack([proj[t], proj[max(t - 4, 0)], proj[0]]).to(device)
        pos = torch.tensor([t, max(t - 4, 0), 0], dtype=torch.int32, device=device)
        slots = torch.tensor([2, 0 if t >= 4 else -1, -1], dtype=torch.int32, device=device)
        o = mixers.short_conv(rows, off, C, w.t().contiguous().to(device), state, slots, None, pos, act)
        outs.append(o[0])
        if t >= 4:
            assert close(o[1], want[t - 4])
    assert close(torch.stack(outs), want)


@pytest.mark.parametrize("device", DEVICES)
def test_short_conv_unequal_sequences_in_one_step(device):
    from ai_agent_kubectl_amd.ops import mixers

    g = torch.Generator().manual_seed(5)
    C, taps = 6, 4
    w = torch.randn(C, taps, generator=g)
    seqs = [torch.randn(n, C, generator=g) for n in (9, 1, 14)]
    want = [oracle.short_conv(s.double().numpy(), w.double().numpy()) for s in seqs]
    state = torch.randn(5, taps - 1, C, generator=g).to(device)
    slots = torch.tensor([4, 0, 2], dtype=torch.int32, device=device)
    got = [[], [], []]
    for lo, hi in ((0, 2), (2, 3), (3, 14)):                    # every sequence advances by what it still has
        parts = [s[lo:hi] for s in seqs]
        lens = [p.shape[0] for p in parts]
        pos = torch.cat([torch.arange(lo, lo + n) for n in lens]).to(torch.int32).to(device)
        o = mixers.short_conv(torch.cat(parts).to(device), 0, C, w.t().contiguous().to(device), state, slots, _seq_meta(lens, device), pos, False)
        at = 0
        for i, n in enumerate(lens):
            got[i].append(o[at:at + n])
            at += n
    for i in range(3):
        assert close(torch.cat(got[i]), want[i])


def _rot_spec(dims, scaling):
    from ai_agent_kubectl_amd.models.config import RotarySpec

    return RotarySpec(dims, 10000.0, *scaling) if scaling else RotarySpec(dims, 10000.0)


@pytest.mark.parametrize("dims,scaling", [(8, None), (32, (6.0, 2048, 24.0, 1.0)), (16, (4.0, 64, 8.0, 1.0)), (6, (40.0, 4096, 2.0, 1.5)),
                                          (64, (2.0, 100000, 32.0, 1.0))])
def test_yarn_frequency_table(dims, scaling):
    f, mag = _rot_spec(dims, scaling).frequencies()
    sc = dict(zip(("factor", "original", "fast", "slow"), scaling)) if scaling else None
    wf, wmag = oracle.rotary_table(dims, 10000.0, sc)
    assert np.allclose(f, wf, rtol=1e-12) and abs(mag - wmag) < 1e-12
    if scaling:
        assert mag > 1.0 and f[-1] <= wf[-1]


class Paged:
    """A paged cache for one attention layer with the pages of each sequence handed out in a scrambled order."""

    def __init__(self, G, D, Dv, lens, device, dtype=torch.float32, seed=0):
        need = [(n + BS - 1) // BS for n in lens]
        nb = sum(need) + 3
        perm = torch.randperm(nb, generator=torch.Generator().manual_seed(seed)).tolist()
        self.k = torch.full((nb, G, BS, D), 7.0, dtype=dtype, device=device)       # whatever a page held before
        self.v = torch.full((nb, G, Dv, BS), -7.0, dtype=dtype, device=device)
        self.tables = torch.zeros((len(lens), max(need)), dtype=torch.int32)
        for i, n in enumerate(need):
            self.tables[i, :n] = torch.tensor([perm.pop() for _ in range(n)], dtype=torch.int32)
        self.device = device

    def slots(self, seq, positions):
        return torch.tensor([int(self.tables[seq, p // BS]) * BS + p % BS for p in positions], dtype=torch.int32, device=self.device)


def _attend(device, q, k, v, m, cuts, gate=None, dtype=torch.float32):
    """q [T, H, D], k [T, G, D], v [T, G, Dv] already rotated: through rope_append (rotation off) and sliding_attention
    in portions `cuts` (a portion of one row after the first runs the decode form).  -> [T, H * Dv]."""
    from ai_agent_kubectl_amd.ops import mixers

    T, H, D = q.shape
    G, Dv = k.shape[1], v.shape[2]
    pg = Paged(G, D, Dv, [T], device, dtype)
    rows = torch.cat([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], dim=1).to(dtype).to(device)
    out, at = [], 0
    for c in cuts:
        pos = list(range(at, at + c))
        p = torch.tensor(pos, dtype=torch.int32, device=device)
        sl = pg.slots(0, pos)
        qq = mixers.rope_append(rows[at:at + c].contiguous(), None, 1.0, p, sl, pg.k, pg.v, H, G, D, Dv, 0)
        decode = c == 1 and at > 0
        gs = gate[at:at + c].contiguous().to(dtype).to(device) if gate is not None else None
        out.append(mixers.sliding_attention(qq, pg.k, pg.v, pg.tables.to(device), None if decode else _seq_meta([c], device), p, sl,
                                            gs, 2 if gate is not None else 0, m["window"], m["keep_first"], m["scale"], max_q=c))
        at += c
    return torch.cat(out)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,G,D,Dv,window,keep", [(4, 2, 16, 8, 8, 2), (3, 1, 10, 7, 21, 5), (2, 2, 12, 20, 1, 0), (1, 1, 8, 8, 0, 0),
                                                  (6, 2, 64, 128, 36, 5), (8, 1, 32, 16, 3, 9), (4, 4, 5, 3, 17, 16),
                                                  (20, 1, 4, 4, 5, 2), (12, 1, 16, 256, 9, 3)])
def test_sliding_attention_windows_and_groups(device, H, G, D, Dv, window, keep):
    g = torch.Generator().manual_seed(H * 100 + D)
    T = 70
    q, k, v = torch.randn(T, H, D, generator=g), torch.randn(T, G, D, generator=g), torch.randn(T, G, Dv, generator=g)
    gate = torch.randn(T, H + 5, generator=g) * 2
    m = dict(window=window, keep_first=keep, scale=0.3)
    want = oracle.window_attention(q.double().numpy(), k.double().numpy(), v.double().numpy(), 0.3, window or T + 1, keep)
    want = (want * oracle.sigmoid(gate.double().numpy()[:, 2:2 + H])[:, :, None]).reshape(T, H * Dv)
    for cuts in ([T], [33] + [1] * 37, [2, 2, 14, 1, 17, 3, 30, 1]):
        assert close(_attend(device, q, k, v, m, cuts, gate), want, 1e-4, 1e-5), cuts


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("decode", [False, True])
@pytest.mark.parametrize("key,seen", [(60 - 11, True), (60 - 12, False), (3, True), (4, False), (0, True)])
def test_window_edges_one_score_stands_out(device, decode, key, seen):
    """Window 12, first 4 tokens kept, query at position 60: one key gets a score far above all others and a value
    of its own; it must carry the result when it is the last key inside the window or the last kept one, and be
    absent one position further out, in a prompt row as in a decoded row."""
    g = torch.Generator().manual_seed(key)
    T, D, Dv, qpos = 61, 8, 4, 60
    q, k, v = torch.randn(T, 1, D, generator=g) * 0.1, torch.randn(T, 1, D, generator=g) * 0.1, torch.randn(T, 1, Dv, generator=g)
    q[qpos, 0], k[key, 0] = 0.0, 0.0
    q[qpos, 0, 0], k[key, 0, 0] = 8.0, 8.0
    v[key, 0] = torch.tensor([100.0, -100.0, 50.0, 25.0])
    m = dict(window=12, keep_first=4, scale=1.0)
    out = _attend(device, q, k, v, m, [qpos, 1] if decode else [T])[qpos].cpu()
    want = oracle.window_attention(q.double().numpy(), k.double().numpy(), v.double().numpy(), 1.0, 12, 4)[qpos, 0]
    assert np.allclose(out.double().numpy(), want, rtol=1e-4, atol=1e-4)
    assert (abs(float(out[0]) - 100.0) < 1.0) == seen


def _delta_inputs(g, T, H, G, D, Dv, channel):
    cv = torch.randn(T, 2 * G * D + H * Dv + 3, generator=g)
    beta_src = torch.randn(T, H + 4, generator=g) * 2
    a_src = torch.randn(T, (H * D if channel else H) + 2, generator=g) * 2
    A_log, dt_bias = torch.randn(H, generator=g) * 0.5, torch.randn(H * D if channel else H, generator=g) - 2.0
    return cv, beta_src, a_src, A_log, dt_bias


def _delta_oracle(cv, beta_src, a_src, A_log, dt_bias, H, G, D, Dv, channel):
    T = cv.shape[0]
    c = cv.double().numpy()
    q, k = c[:, :G * D].reshape(T, G, D), c[:, G * D:2 * G * D].reshape(T, G, D)
    q = q / np.sqrt((q * q).sum(-1, keepdims=True) + 1e-6) * D ** -0.5
    k = k / np.sqrt((k * k).sum(-1, keepdims=True) + 1e-6)
    v = c[:, 2 * G * D:2 * G * D + H * Dv].reshape(T, H, Dv)
    beta = oracle.sigmoid(beta_src.double().numpy()[:, 1:1 + H])
    n = H * D if channel else H
    sp = oracle.softplus(a_src.double().numpy()[:, 2:2 + n] + dt_bias.double().numpy())
    rate = np.exp(A_log.double().numpy())
    decay = np.exp(-rate[None, :, None] * sp.reshape(T, H, D)) if channel else np.repeat(np.exp(-rate[None] * sp)[:, :, None], D, 2)
    rep = H // G
    return oracle.delta_rule(np.repeat(q, rep, 1), np.repeat(k, rep, 1), v, beta, decay).reshape(T, H * Dv)


def _delta_run(device, inputs, H, G, D, Dv, channel, cuts, S, slot):
    from ai_agent_kubectl_amd.ops import mixers

    cv, beta_src, a_src, A_log, dt_bias = [t.to(device) for t in inputs]
    out, at = [], 0
    for c in cuts:
        sl = slice(at, at + c)
        pos = torch.arange(at, at + c, dtype=torch.int32, device=device)
        qk, beta, decay = mixers.delta_prep(cv[sl].contiguous(), beta_src[sl].contiguous(), 1, a_src[sl].contiguous(), 2, A_log,
                                            dt_bias, H, G, D, channel)
        decode = c == 1 and at > 0
        slots = torch.tensor([slot], dtype=torch.int32, device=device)
        out.append(mixers.delta_scan(qk, cv[sl].contiguous(), 2 * G * D, beta, decay, S, slots, None if decode else _seq_meta([c], device),
                                     pos, H, G, D, Dv))
        at += c
    return torch.cat(out)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("channel", [False, True])
@pytest.mark.parametrize("H,G,D,Dv", [(2, 1, 8, 12), (1, 1, 5, 19), (3, 3, 33, 16), (4, 2, 64, 70), (2, 2, 130, 8)])
def test_delta_rule_recurrence(device, channel, H, G, D, Dv):
    """Whole, row by row through the decode form, and in portions; the slot holds another sequence's memory first."""
    g = torch.Generator().manual_seed(D + Dv)
    T = 40
    inputs = _delta_inputs(g, T, H, G, D, Dv, channel)
    want = _delta_oracle(*inputs, H, G, D, Dv, channel)
    final = None
    for cuts in ([T], [1] * T, [2, 2, 3, 9, 2, 16, 1, 1, 4]):
        S = torch.randn(3, H, Dv, D, generator=g).to(device) * 30
        got = _delta_run(device, inputs, H, G, D, Dv, channel, cuts, S, 1)
        assert close(got, want, 2e-4, 2e-5), cuts
        final = S[1].cpu() if final is None else final
        assert torch.allclose(S[1].cpu(), final, rtol=1e-4, atol=1e-5)      # the memory after the last row does not depend on the cuts


@pytest.mark.parametrize("device", DEVICES)
def test_delta_rule_keeps_a_far_token_and_overwrites_on_the_same_key(device):
    """A value written at row 2 with beta near 1 under a decay near 1 is read back 300 rows later through the same
    key among rows whose keys are orthogonal to it; a second write on that key replaces it instead of adding."""
    H = G = 1
    D, Dv, T = 8, 4, 320
    g = torch.Generator().manual_seed(1)
    cv = torch.zeros(T, 2 * D + Dv + 3)
    cv[:, D + 1:2 * D] = torch.randn(T, D - 1, generator=g)        # keys of the other rows: no part along entry 0
    cv[:, 2 * D:2 * D + Dv] = torch.randn(T, Dv, generator=g)
    for t, val in ((2, [9.0, -3.0, 5.0, 1.0]), (150, [-4.0, 8.0, 0.5, 2.0])):
        cv[t, D:2 * D] = 0.0
        cv[t, D] = 3.0
        cv[t, 2 * D:2 * D + Dv] = torch.tensor(val)
    cv[310, :D] = 0.0
    cv[310, 0] = 2.0                                                # the query at row 310 asks along entry 0
    cv[310, D:2 * D] = 0.0
    cv[310, D + 1] = 1.0
    beta_src = torch.full((T, 5), -20.0)                            # the other rows write almost nothing
    beta_src[2, 1] = beta_src[150, 1] = 20.0
    a_src, A_log, dt_bias = torch.zeros(T, 3), torch.zeros(1), torch.tensor([-18.0])
    inputs = (cv, beta_src, a_src, A_log, dt_bias)
    want = _delta_oracle(*inputs, H, G, D, Dv, False)
    S = torch.zeros(1, H, Dv, D).to(device)
    got = _delta_run(device, inputs, H, G, D, Dv, False, [200] + [1] * 120, S, 0).cpu().double().numpy()
    assert np.allclose(got, want, rtol=1e-4, atol=1e-5)
    assert np.allclose(got[310], np.array([-4.0, 8.0, 0.5, 2.0]) * D ** -0.5, atol=1e-3)   # the second write alone


# ---------------------------------------------------------------------------------------------------
# the model through the engine
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", VARIANTS)
def test_whole_prompt(tmp_path, device, name):
    c, W, path = model_for(tmp_path, name)
    toks = tokens_for(c, 45, seed=1)
    sess = session(path, device)
    assert rel_err(replay(sess, toks, [45]), want_logits(c, W, toks)) < tol("float32")
    one = tokens_for(c, 1, seed=2)                      # a sequence of one token: nothing before it anywhere
    assert rel_err(replay(sess, one, [1], rid="one"), want_logits(c, W, one)) < tol("float32")


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", ["base", "attention_first"])
def test_layer_trail(tmp_path, device, name):
    c, W, path = model_for(tmp_path, name, seed=2)
    toks = tokens_for(c, 20, seed=3)
    trail = []
    want_logits(c, W, toks, trail)
    sess = session(path, device)
    got = []
    sess.runner.model.layer_hook = lambda i, x: got.append(x.detach().cpu().double().numpy().copy())
    replay(sess, toks, [20])
    assert len(got) == len(trail) == len(c["layers"])
    for i, (a, b) in enumerate(zip(got, trail)):
        assert np.abs(a[:20] - b).max() < 2e-4 * max(1.0, np.abs(b).max()), i


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", VARIANTS)
def test_decode_token_by_token(tmp_path, device, name):
    """10 prompt tokens, then 60 decoded one by one: over page borders, past every window and kept span."""
    c, W, path = model_for(tmp_path, name, seed=3)
    toks = tokens_for(c, 70, seed=4)
    sess = session(path, device)
    assert rel_err(replay(sess, toks, [10] + [1] * 60), want_logits(c, W, toks)) < tol("float32")


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name,cuts", [("base", [2, 2, 3, 9, 2, 16, 1, 1, 15, 2]), ("attention_first", [5, 5, 2, 11, 17, 13]),
                                       ("keep_all", [1, 2, 2, 2, 2, 2, 30, 2, 10]), ("no_window", [16, 16, 2, 14, 5])])
def test_portions(tmp_path, device, name, cuts):
    c, W, path = model_for(tmp_path, name, seed=5)
    toks = tokens_for(c, sum(cuts), seed=6)
    sess = session(path, device)
    assert rel_err(replay(sess, toks, cuts), want_logits(c, W, toks)) < tol("float32")


@pytest.mark.parametrize("device", DEVICES)
def test_mixed_batches_pages_and_slots_reused(tmp_path, device):
    """Six unequal requests through a pool of 112 tokens and 3 state slots: portions of some beside single tokens
    of others; a finished request's pages and slot go to the next one, whose memories and conv inputs must start
    from zero."""
    c, W, path = model_for(tmp_path, "base", seed=4)
    sess = session(path, device, max_tokens=112, max_requests=3)
    lens = {"a": 40, "b": 9, "c": 33, "d": 21, "e": 30, "f": 17}
    toks = {k: tokens_for(c, n, seed=10 + i) for i, (k, n) in enumerate(lens.items())}
    want = {k: want_logits(c, W, v) for k, v in toks.items()}
    plan = [[("a", 7)], [("a", 2), ("b", 3)], [("a", 1), ("b", 1), ("c", 20)], [("a", 14), ("b", 1), ("c", 2)],
            [("b", 4), ("c", 1), ("a", 1)], [("c", 10), ("a", 15)], [("d", 21)], [("d", 0), ("e", 2)],
            [("e", 27), ("f", 16)], [("e", 1), ("f", 1)]]
    at = {k: 0 for k in lens}
    got = {k: [] for k in lens}
    for step in plan:
        entries, end = [], []
        for rid, n in step:
            if n == 0:
                continue
            part = toks[rid][at[rid]:at[rid] + n]
            entries.append({"id": rid, "tokens": part, "want": list(range(n))})
            at[rid] += n
            if at[rid] == lens[rid]:
                end.append(rid)
        out = sess.step(entries, end)
        o = 0
        for e in entries:
            got[e["id"]].append(out[o:o + len(e["tokens"])])
            o += len(e["tokens"])
    assert at == lens
    assert sess.sched.state_slots.num_free == 3 and sess.sched.bm.num_free == sess.sched.bm.num_blocks
    for k in lens:
        assert rel_err(np.concatenate(got[k]), want[k]) < tol("float32"), k


@pytest.mark.parametrize("device", DEVICES)
def test_batch_against_each_alone(tmp_path, device):
    """Three unequal requests decoded together give what each gives alone, to rounding."""
    c, W, path = model_for(tmp_path, "attention_first", seed=7)
    toks = [tokens_for(c, n, seed=40 + n) for n in (30, 12, 23)]
    alone = [replay(session(path, device), t, [len(t) - 6] + [1] * 6) for t in toks]
    sess = session(path, device)
    got = [[] for _ in toks]
    for i, t in enumerate(toks):
        got[i].append(sess.step([{"id": str(i), "tokens": t[:-6], "want": list(range(len(t) - 6))}], []))
    for d in range(6):
        out = sess.step([{"id": str(i), "tokens": [t[len(t) - 6 + d]], "want": [0]} for i, t in enumerate(toks)], [])
        for i in range(3):
            got[i].append(out[i:i + 1])
    for i in range(3):
        assert rel_err(np.concatenate(got[i]), alone[i]) < 2e-5


@pytest.mark.parametrize("device", DEVICES)
def test_long_decode_and_a_window_over_many_pages(tmp_path, device):
    """A 150-position window with 20 kept tokens over a 400-token sequence, the last 230 decoded one by one."""
    c = make_config([parallel_layer(left=attention_cfg(heads=2, kv_heads=1, dim=8, vdim=8, window=150, keep_first=20, rot_dims=8,
                                                       scaling=(8.0, 128, 16.0, 1.0)), ff=16), delta_layer(ff=0)], width=16, vocab=64, side=2)
    W = oracle.random_tensors(c, 9)
    path = write_checkpoint(tmp_path / "long", c, W)
    toks = tokens_for(c, 400, seed=8)
    sess = session(path, device, max_tokens=448)
    assert rel_err(replay(sess, toks, [170] + [1] * 230), want_logits(c, W, toks)) < tol("float32")


@pytest.mark.parametrize("device", DEVICES)
def test_steps_that_want_nothing(tmp_path, device):
    c, W, path = model_for(tmp_path, "base", seed=8)
    toks = tokens_for(c, 30, seed=9)
    sess = session(path, device)
    assert sess.step([{"id": "r", "tokens": toks[:12], "want": []}], []).shape == (0, c["vocab"])
    assert sess.step([{"id": "r", "tokens": toks[12:13], "want": []}], []).shape == (0, c["vocab"])
    got = sess.step([{"id": "r", "tokens": toks[13:], "want": [0, 16]}], ["r"])
    assert rel_err(got, want_logits(c, W, toks)[[13, 29]]) < tol("float32")


@pytest.mark.parametrize("device", DEVICES)
def test_generate_greedy_through_scheduler(tmp_path, device):
    """Greedy generation through build_engine / generate_blocking: the scheduler chunks the prompts (12 tokens a
    step), admits at most as many requests as there are state slots and frees slots for the ones that wait."""
    from ai_agent_kubectl_amd.engine.builder import EngineOptions, build_engine
    from ai_agent_kubectl_amd.engine.sequence import SamplingParams

    c, W, path = model_for(tmp_path, "base", seed=6)
    prompts = [tokens_for(c, n, seed=20 + n) for n in (5, 19, 1, 26, 8, 13)]
    eng = build_engine(EngineOptions(model=path, device=device, dtype="float32", max_batch=3, max_batched_tokens=12,
                                     max_model_len=64, kv_cache_tokens=256, graph_buckets=(1, 2, 3), use_graphs=False,
                                     safe_decode=False, ignore_eos=True))
    assert eng.scheduler.state_slots.num_slots == 3 and not eng.bm.prefix_caching
    seqs = eng.generate_blocking(prompts, SamplingParams(max_new_tokens=10, ignore_eos=True, safe_decode=False))
    for p, s in zip(prompts, seqs):
        toks = list(p)
        for _ in range(10):
            toks.append(int(np.argmax(want_logits(c, W, toks)[-1])))
        assert s.generated == toks[len(p):]
    assert eng.scheduler.state_slots.num_free == 3


def test_config_reader(tmp_path):
    from ai_agent_kubectl_amd.models.config import SuvapelConfig, get_config

    for name in VARIANTS:
        c, W, path = model_for(tmp_path, name)
        cfg = get_config(path)
        assert cfg.family == "suvapel" and cfg.num_layers == len(c["layers"]) and cfg.has_state
        assert SuvapelConfig.from_dict(cfg.to_dict(), cfg.name) == cfg
    cfg = get_config(model_for(tmp_path, "no_window")[2])
    a = cfg.layers[0].attention
    assert a.window == 0 and a.rot.dims == 0 and a.conv == 1 and cfg.layers[0].delta.channel_decay
    bad = variant("base")
    bad["layers"][0]["type"] = "convolution"
    with pytest.raises(ValueError):
        SuvapelConfig.from_dict(bad)
    bad = variant("base")
    bad["layers"][1]["mixer"]["left"]["kv_heads"] = 3          # 4 heads in groups of 3
    with pytest.raises(ValueError):
        SuvapelConfig.from_dict(bad)
    bad = variant("base")
    bad["layers"][0]["mlp"]["kind"] = "experts"
    with pytest.raises(ValueError):
        SuvapelConfig.from_dict(bad)
    cfg = get_config("tiny-suvapel")
    assert cfg.kv_bytes_per_token() == 2 * 2 * (32 + 32) * 2 and cfg.state_bytes_per_slot() > 0


def test_loader_checks_shapes(tmp_path):
    from ai_agent_kubectl_amd.models.config import get_config
    from ai_agent_kubectl_amd.models.weights import ParallelInfo, build_weights, suvapel_random_weights

    c, W, path = model_for(tmp_path, "base")
    W2 = dict(W)
    W2["l1.mix.right.a2"] = W["l1.mix.right.a2"][:-1]
    bad = write_checkpoint(tmp_path / "bad", c, W2)
    with pytest.raises((ValueError, RuntimeError)):
        build_weights(bad, get_config(bad), ParallelInfo(), dtype=torch.float32)
    del W2["l1.mix.right.a2"]
    bad = write_checkpoint(tmp_path / "bad2", c, W2)
    with pytest.raises(KeyError):
        build_weights(bad, get_config(bad), ParallelInfo(), dtype=torch.float32)
    cfg = get_config("tiny-suvapel")
    Wr = suvapel_random_weights(cfg, seed=1, dtype=torch.float32)
    assert Wr["layers.1.w_a2"].shape == (4 * 32, 8) and Wr["layers.0.w_in"].shape[1] == 128


# ---------------------------------------------------------------------------------------------------
# GPU only: the bf16 engine, wider shapes, captured decode
@pytest.mark.gpu
@pytest.mark.parametrize("name", ["base", "attention_first"])
def test_bf16_engine(tmp_path, name):
    c, W, path = model_for(tmp_path, name, seed=12)
    toks = tokens_for(c, 60, seed=13)
    want = want_logits(c, W, toks)
    sess = session(path, "cuda", dtype="bfloat16")
    assert rel_err(replay(sess, toks, [60]), want) < tol("bfloat16")
    assert rel_err(replay(sess, toks, [7, 2, 20, 1, 1, 1, 12, 16], rid="p"), want) < tol("bfloat16")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_wider_shapes_gpu(tmp_path, dtype):
    """Head sizes 128 / 64 with 8 query heads per key/value head, a 256-wide feed-forward, 100 tokens in portions."""
    c = make_config([parallel_layer(left=attention_cfg(heads=8, kv_heads=1, dim=128, vdim=64, conv=4, window=48, keep_first=4, rot_dims=64,
                                                       scaling=(16.0, 512, 32.0, 1.0)),
                                    right=delta_mixer_cfg(heads=4, kv_heads=2, dim=128, vdim=128, conv=4), ff=256),
                     delta_layer(heads=4, kv_heads=4, dim=64, vdim=96, conv=4, ff=256)], width=256, vocab=512, side=32)
    W = oracle.random_tensors(c, 14, rank=20)
    path = write_checkpoint(tmp_path / "wide", c, W)
    toks = tokens_for(c, 100, seed=15)
    want = want_logits(c, W, toks)
    sess = session(path, "cuda", dtype=dtype)
    assert rel_err(replay(sess, toks, [64, 2, 1, 1, 30, 1, 1]), want) < tol(dtype)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_graph_decode_matches_eager(tmp_path, dtype):
    """Decode steps replayed from captured graphs (several replays with eager prefill steps between them) give
    the tokens of the eager engine."""
    from ai_agent_kubectl_amd.engine.builder import EngineOptions, build_engine
    from ai_agent_kubectl_amd.engine.sequence import SamplingParams

    c, W, path = model_for(tmp_path, "base", seed=11)
    prompts = [tokens_for(c, n, seed=30 + n) for n in (7, 21, 3, 12, 9)]
    got = []
    for graphs in (False, True):
        eng = build_engine(EngineOptions(model=path, device="cuda", dtype=dtype, max_batch=4, max_model_len=96,
                                         kv_cache_tokens=512, graph_buckets=(1, 2, 4), use_graphs=graphs, safe_decode=False,
                                         ignore_eos=True))
        if graphs:
            eng.runner.capture_graphs(autotune=False)
            assert eng.runner.graphs
        seqs = eng.generate_blocking(prompts, SamplingParams(max_new_tokens=24, ignore_eos=True, safe_decode=False))
        got.append([s.generated for s in seqs])
        if graphs:
            assert eng.runner.stats["graph_replays"] > 0
    assert got[0] == got[1]


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,D,Dv,window,keep", [(4, 1, 64, 64, 44, 7), (6, 2, 64, 128, 36, 5), (8, 2, 128, 128, 100, 20), (2, 2, 128, 64, 0, 0),
                                                  (8, 1, 256, 256, 17, 33), (4, 4, 64, 256, 1, 0), (3, 1, 128, 128, 16, 16)])
def test_sliding_attention_matrix_core_kernel(H, G, D, Dv, window, keep):
    """bf16 prompt portions run on the matrix cores: against the oracle on the bf16-rounded inputs, whole and in
    portions whose rows start anywhere in a page; the vector kernel agrees."""
    from ai_agent_kubectl_amd.ops import mixers

    g = torch.Generator().manual_seed(H + D + window)
    T = 150
    bf = lambda t: t.to(torch.bfloat16).float()
    q, k, v = bf(torch.randn(T, H, D, generator=g)), bf(torch.randn(T, G, D, generator=g)), bf(torch.randn(T, G, Dv, generator=g))
    gate = bf(torch.randn(T, H + 5, generator=g) * 2)
    m = dict(window=window, keep_first=keep, scale=D ** -0.5 * 2)
    want = oracle.window_attention(q.double().numpy(), k.double().numpy(), v.double().numpy(), m["scale"], window or T + 1, keep)
    want = (want * oracle.sigmoid(gate.double().numpy()[:, 2:2 + H])[:, :, None]).reshape(T, H * Dv)
    assert mixers.require_mixers().ka_sliding_attention_tile_ok(H, G, D, Dv, BS)
    outs = []
    for tile in (True, False):
        mixers.SLIDING_TILE = tile
        try:
            for cuts in ([T], [37, 9, 70, 1, 33], [16, 16, 8, 110]):
                got = _attend("cuda", q, k, v, m, cuts, gate, dtype=torch.bfloat16)
                assert close(got, want, 2e-2, 2e-2), (tile, cuts)
                outs.append(got.float().cpu())
        finally:
            mixers.SLIDING_TILE = True
    assert (outs[0] - outs[3]).abs().max() < 2e-2


@pytest.mark.gpu
@pytest.mark.parametrize("key,seen", [(140 - 43, True), (140 - 44, False), (6, True), (7, False), (0, True)])
def test_window_edges_on_the_matrix_cores(key, seen):
    """Window 44, first 7 tokens kept, the query at position 140 inside a 150-row prompt portion (bf16, head size 64):
    the key whose score stands out carries the result exactly when the mask lets it."""
    g = torch.Generator().manual_seed(key)
    T, D, Dv, qpos = 150, 64, 64, 140
    q, k, v = torch.randn(T, 2, D, generator=g) * 0.05, torch.randn(T, 1, D, generator=g) * 0.05, torch.randn(T, 1, Dv, generator=g)
    q[qpos], k[key] = 0.0, 0.0
    q[qpos, :, 0], k[key, 0, 0] = 8.0, 8.0
    v[key, 0] = 100.0
    m = dict(window=44, keep_first=7, scale=1.0)
    out = _attend("cuda", q, k, v, m, [T], dtype=torch.bfloat16)[qpos].float().cpu()
    assert (abs(float(out[0]) - 100.0) < 2.0) == seen and (abs(float(out[Dv]) - 100.0) < 2.0) == seen


@pytest.mark.gpu
def test_mixed_steps_on_the_matrix_cores(tmp_path):
    """bf16 engine with head sizes the matrix-core attention takes: single decoded rows of two requests ahead of a
    prompt portion of a third in one step (the decoded rows go through the vector kernel, the portion through the
    tile kernel), then the roles change."""
    c = make_config([parallel_layer(left=attention_cfg(heads=4, kv_heads=2, dim=64, vdim=64, window=24, keep_first=3, rot_dims=32),
                                    right=delta_mixer_cfg(heads=2, kv_heads=1, dim=32, vdim=32, conv=4), ff=64), delta_layer(ff=32)],
                    width=64, vocab=128, side=8)
    W = oracle.random_tensors(c, 21)
    path = write_checkpoint(tmp_path / "mixed", c, W)
    toks = {k: tokens_for(c, n, seed=50 + n) for k, n in (("a", 44), ("b", 37), ("c", 90))}
    want = {k: want_logits(c, W, v) for k, v in toks.items()}
    sess = session(path, "cuda", dtype="bfloat16", max_tokens=256)
    plan = [[("a", 40), ("b", 35)], [("a", 1), ("b", 1), ("c", 50)], [("a", 1), ("c", 1), ("b", 1)], [("c", 37), ("a", 1)],
            [("c", 1), ("a", 1)], [("c", 1)]]
    at, got = {k: 0 for k in toks}, {k: [] for k in toks}
    for step in plan:
        entries = []
        for rid, n in step:
            entries.append({"id": rid, "tokens": toks[rid][at[rid]:at[rid] + n], "want": list(range(n))})
            at[rid] += n
        out = sess.step(entries, [rid for rid, _ in step if at[rid] == len(toks[rid])])
        o = 0
        for e in entries:
            got[e["id"]].append(out[o:o + len(e["tokens"])])
            o += len(e["tokens"])
    for k in toks:
        assert at[k] == len(toks[k]) and rel_err(np.concatenate(got[k]), want[k]) < tol("bfloat16"), k


@pytest.mark.gpu
@pytest.mark.parametrize("lanes", [4, 8, 16])
@pytest.mark.parametrize("H,G,D,Dv,channel", [(2, 1, 64, 70, True), (3, 3, 33, 16, False), (2, 2, 128, 40, True), (1, 1, 200, 64, False)])
def test_delta_rule_lanes_per_column(lanes, H, G, D, Dv, channel):
    """The kernel's forms with 4, 8 and 16 lanes per memory column give the oracle's result."""
    from ai_agent_kubectl_amd.ops import mixers

    g = torch.Generator().manual_seed(D + lanes)
    inputs = _delta_inputs(g, 50, H, G, D, Dv, channel)
    want = _delta_oracle(*inputs, H, G, D, Dv, channel)
    mixers.DELTA_LANES = lanes
    try:
        for cuts in ([50], [20] + [1] * 30):
            S = torch.randn(2, H, Dv, D, generator=g).cuda()
            assert close(_delta_run("cuda", inputs, H, G, D, Dv, channel, cuts, S, 1), want, 2e-4, 2e-5), cuts
    finally:
        mixers.DELTA_LANES = 0


@pytest.mark.gpu
@pytest.mark.parametrize("taps,act", [(4, True), (3, False), (2, True)])
def test_short_conv_many_rows_in_bf16(taps, act):
    """Steps of 1024 rows and more in bf16 take eight channels per thread: two sequences that continue from their
    slots (one of them from position 1: a zero before the start), against the oracle on the same bf16 inputs."""
    from ai_agent_kubectl_amd.ops import mixers

    g = torch.Generator().manual_seed(taps)
    C, off, lens, first = 136, 16, [700, 500], [40, 1]
    w = torch.randn(C, taps, generator=g)
    seqs = [torch.randn(f + n, C, generator=g).to(torch.bfloat16) for f, n in zip(first, lens)]
    want = [oracle.short_conv(s.double().numpy(), w.double().numpy()) for s in seqs]
    state = torch.zeros(3, taps - 1, C, dtype=torch.bfloat16).cuda()
    slots = torch.tensor([2, 0], dtype=torch.int32).cuda()
    wt = w.t().contiguous().cuda()
    outs = []
    for lo_hi in ([(0, first[0]), (0, first[1])], [(first[0], first[0] + lens[0]), (first[1], first[1] + lens[1])]):
        parts = [s[a:b] for s, (a, b) in zip(seqs, lo_hi)]
        rows = torch.zeros(sum(p.shape[0] for p in parts), C + 24, dtype=torch.bfloat16)
        rows[:, off:off + C] = torch.cat(parts)
        pos = torch.cat([torch.arange(a, b) for a, b in lo_hi]).to(torch.int32).cuda()
        outs.append(mixers.short_conv(rows.cuda(), off, C, wt, state, slots, _seq_meta([b - a for a, b in lo_hi], "cuda"), pos, act))
    got = outs[1].float().cpu().double().numpy()
    ref = np.concatenate([w_[f:] for w_, f in zip(want, first)])
    ref = oracle.silu(ref) if act else ref
    assert np.allclose(got, ref, rtol=2e-2, atol=2e-2)
