"""Zibinex in the engine against the plain oracle (tests/zibinex_oracle.py).

Every test makes its own small configuration and random (or crafted) weights, writes them as a checkpoint folder
(config.json + model.safetensors: the reader and the loader are under test too), builds the engine on it and compares
logits with the oracle's whole-sequence forward.  The same bodies run on the CPU (the ops' torch references) and,
marked `gpu`, on the HIP kernels in fp32 and bf16.
"""
import json
import os

import numpy as np
import pytest
import torch

import zibinex_oracle as oracle
from zibinex_oracle import attention_layer, latent_layer, make_config, shared

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
BS = 16


def write_checkpoint(path, config, W):
    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(config, f)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in W.items()}, os.path.join(path, "model.safetensors"))
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


def run_plan(sess, toks, plan):
    """plan: steps of (request, tokens to feed); a request ends with its last token.  -> logits per request."""
    at, got = {k: 0 for k in toks}, {k: [] for k in toks}
    for step in plan:
        entries, end = [], []
        for rid, n in step:
            entries.append({"id": rid, "tokens": toks[rid][at[rid]:at[rid] + n], "want": list(range(n))})
            at[rid] += n
            if at[rid] == len(toks[rid]):
                end.append(rid)
        out = sess.step(entries, end)
        o = 0
        for e in entries:
            got[e["id"]].append(out[o:o + len(e["tokens"])])
            o += len(e["tokens"])
    assert all(at[k] == len(toks[k]) for k in toks)
    return {k: np.concatenate(v) for k, v in got.items()}


def rel_err(got, want):
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    w = want - want.mean(-1, keepdims=True)
    return float(np.sqrt((d ** 2).mean(-1)).max() / np.sqrt((w ** 2).mean()))


def tol(dtype):
    return 2e-4 if dtype == "float32" else 6e-2


def ok_bf16(got, want):
    """bf16 engine against the float64 oracle, position by position: the typical position within 3 %, none beyond
    12 % (these tiny widths amplify a rounding; a wrong key, window or state is far beyond both)."""
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    w = want - want.mean(-1, keepdims=True)
    e = np.sqrt((d ** 2).mean(-1)) / np.sqrt((w ** 2).mean())
    return bool(np.median(e) < 3e-2 and e.max() < 0.12)


def all_experts(config):
    """The same model with every expert chosen: bf16 runs are compared on it, because a rounding that flips a close
    choice between two experts changes a token's result by far more than a rounding does."""
    out = json.loads(json.dumps(config))
    for L in out["layers"]:
        if L.get("mlp") and L["mlp"]["kind"] == "moe":
            L["mlp"]["router"]["top"] = L["mlp"]["router"]["experts"]
    return out


def tokens_for(config, n, seed=0):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, config["vocab"], (n,), generator=g).tolist()


def want_logits(config, W, tokens, layer_out=None):
    return oracle.forward(config, oracle.as_arrays(W), tokens, layer_out)


def variant(name):
    if name == "base":           # both mixers, all three feed-forwards, a shared layer; window 8 is half a page
        return make_config([latent_layer(mlp="dense"), attention_layer(), latent_layer(), attention_layer(mlp=None),
                            shared(latent_layer(), 2)])
    if name == "odd":            # sizes that share no factor: 3 heads over 1 key/value head, 7 / 9 / 11 entries, a window of 21
        # over a page border, three of four experts, rotation without scaling, a shared attention layer that comes
        # BEFORE its owner
        att = attention_layer(heads=3, kv_heads=1, dim=7, vdim=9, window=21, scale=0.3, experts=4, top=3, ff=11)
        return make_config([shared(att, 2), latent_layer(heads=5, dim=3, rot_dim=6, vdim=7, kv_rank=11, scaling=None, mlp="dense",
                                                         ff=13, limit=0.4), att], width=20, vocab=50, eps=1e-3)
    if name == "no_mask":        # attention over every earlier key, no rotation at all, one head, every expert chosen,
        # rotation on a part of the rotated entries, a latent layer with a window of its own
        return make_config([attention_layer(heads=1, kv_heads=1, dim=8, vdim=8, window=0, experts=2, top=2),
                            latent_layer(heads=1, dim=8, rot_dim=4, vdim=8, kv_rank=8, rot_dims=0, mlp=None),
                            latent_layer(heads=2, dim=2, rot_dim=8, vdim=3, kv_rank=6, rot_dims=4, scaling=(16.0, 20, 4.0, 0.5),
                                         window=5, top=1)], width=16, vocab=40)
    if name == "window_one":     # a window of one position (only the token itself), equal head counts, top 1
        return make_config([attention_layer(heads=2, kv_heads=2, dim=4, vdim=6, window=1, top=1),
                            attention_layer(heads=4, kv_heads=4, dim=5, vdim=3, window=17, mlp="dense")], width=12, vocab=32)
    if name == "own_constants":  # layers on another's tensors whose entries differ in what is not a tensor's size: window, scale,
        # rotary table, number of chosen experts
        return make_config([attention_layer(window=8), latent_layer(),
                            shared(attention_layer(window=3, scale=0.9, top=1), 0),
                            shared(latent_layer(window=4, scaling=None, base=50.0, scale=0.2, top=3), 1)])
    raise KeyError(name)


VARIANTS = ["base", "odd", "no_mask", "window_one", "own_constants"]


def model_for(tmp_path, name, seed=0, every_expert=False):
    c = all_experts(variant(name)) if every_expert else variant(name)
    W = oracle.random_tensors(c, seed)
    return c, W, write_checkpoint(tmp_path / name, c, W)


def close(got, want, rtol=1e-4, atol=1e-4):
    return np.allclose(np.asarray(got.detach().float().cpu().double()), np.asarray(want), rtol=rtol, atol=atol)


def _seq_meta(lens, device):
    return torch.tensor(np.concatenate([[0], np.cumsum(lens)]), dtype=torch.int32, device=device)


# ---------------------------------------------------------------------------------------------------
# each mechanism alone: ops.mixers (torch reference on CPU, HIP kernel on GPU) against the oracle
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("width", [24, 100, 513])
def test_one_plus_norms_around_a_sublayer(device, width):
    """The loader keeps 1 + w; the closing pass adds norm(y) to the residual and norms the sum for the next sublayer;
    y may be an fp32 sum (experts) beside bf16-typed results."""
    from ai_agent_kubectl_amd.ops import mixers

    g = torch.Generator().manual_seed(width)
    x, y = torch.randn(5, width, generator=g) * 3 + 1, torch.randn(5, width, generator=g) * 7 - 2
    w1, w2 = torch.rand(width, generator=g) - 0.5, torch.rand(width, generator=g) - 0.5
    eps = 1e-3
    xd = x.clone().to(device)
    h = mixers.group_rmsnorm(xd, (1 + w1).to(device), 1, eps, out_dtype=torch.float32)
    assert close(h, oracle.norm_one_plus(x.double().numpy(), w1.double().numpy(), eps), 1e-5, 1e-5)
    new = x.double().numpy() + oracle.norm_one_plus(y.double().numpy(), w2.double().numpy(), eps)
    h = mixers.post_norm_residual(xd, y.to(device), (1 + w2).to(device), None, (1 + w1).to(device), 1, eps, torch.float32)
    assert close(xd, new, 1e-5, 1e-5) and close(h, oracle.norm_one_plus(new, w1.double().numpy(), eps), 1e-5, 1e-5)
    assert not np.allclose(new, x.double().numpy() + oracle.rms_div(y.double().numpy(), eps) * w2.double().numpy(), atol=1e-2)
    xd = x.clone().to(device)
    assert mixers.post_norm_residual(xd, y.to(device), (1 + w2).to(device), None, None, 1, eps) is None and close(xd, new, 1e-5, 1e-5)
    if device == "cuda":         # an fp32 result, the next norm written in bf16
        xd = x.clone().to(device)
        h = mixers.post_norm_residual(xd, y.to(device), (1 + w2).to(device), None, (1 + w1).to(device), 1, eps, torch.bfloat16)
        assert h.dtype == torch.bfloat16 and close(xd, new, 1e-5, 1e-5)
        assert close(h, oracle.norm_one_plus(new, w1.double().numpy(), eps), 1e-2, 1e-2)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("rows,ff", [(3, 20), (7, 1030)])
def test_clamped_gated_unit(device, rows, ff):
    from ai_agent_kubectl_amd.ops import mixers

    g = torch.Generator().manual_seed(ff)
    gu = torch.randn(rows, 2 * ff, generator=g) * 2        # a good part of the entries lies beyond the limit 0.9
    a, u = gu[:, :ff].double().numpy(), gu[:, ff:].double().numpy()
    a = np.minimum(a, 0.9)
    want = a * oracle.sigmoid(1.702 * a) * (np.clip(u, -0.9, 0.9) + 1.0)
    assert close(mixers.glu_clamp(gu.to(device), 0.9, 1.702), want, 1e-5, 1e-5)
    assert (gu[:, :ff] < -0.9).any() and want.min() < -0.9 * 0.2   # the gate has no lower limit


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,D,Dr,rot,R,scaling", [(3, 6, 4, 4, 12, (4.0, 32, 8.0, 1.0)), (2, 5, 16, 16, 8, (8.0, 64, 32.0, 1.0)),
                                                   (1, 8, 6, 4, 16, None), (4, 2, 8, 0, 5, None)])
def test_interleaved_rotary_direct_queries_and_latent_rows(device, H, D, Dr, rot, R, scaling):
    """The fused row [c | k_r | q | g]: the latent is normed and k_r rotated into the cache row of the token's slot,
    q's rotated parts are rotated in pairs (2i, 2i + 1) with the scaled frequencies and magnitude."""
    from ai_agent_kubectl_amd.models.config import RotarySpec
    from ai_agent_kubectl_amd.ops import mixers

    g = torch.Generator().manual_seed(H * 10 + Dr)
    T, eps = 9, 1e-4
    sc = dict(zip(("factor", "original", "fast", "slow"), scaling)) if scaling else None
    spec = RotarySpec(rot, 50.0, *(scaling or ()))
    f, mag = spec.frequencies() if rot else ([], 1.0)
    if rot:
        wf, wmag = oracle.rotary_table(rot, 50.0, sc)
        assert np.allclose(f, wf, rtol=1e-12) and abs(mag - wmag) < 1e-12
    P = R + Dr + H * (D + Dr) + H + 3
    proj = torch.randn(T, P, generator=g)
    w = torch.rand(R, generator=g) + 0.5
    pos = torch.tensor([0, 1, 2, 17, 18, 100, 101, 4000, 5], dtype=torch.int32)
    cache = torch.full((4, BS, R + Dr), 9.0)
    slots = torch.tensor([16, 17, 18, 1, 2, 36, -1, 63, 5], dtype=torch.int32)
    inv = torch.tensor(f, dtype=torch.float32)
    cd = cache.to(device)
    assert mixers.latent_prep(proj.to(device), 0, R, Dr, None, w.to(device), inv.to(device), pos.to(device), slots.to(device), cd,
                              rot, eps, interleaved=True, mag=mag) is None
    pn = proj.double().numpy()
    c = oracle.rms_div(pn[:, :R], eps) * w.double().numpy()
    kr = oracle.rotate_pairs(pn[:, R:R + Dr], pos.numpy(), np.asarray(f), mag, rot)
    rows = cd.cpu().reshape(-1, R + Dr).double().numpy()
    for t, s in enumerate(slots.tolist()):
        if s >= 0:
            assert np.allclose(rows[s], np.concatenate([c[t], kr[t]]), rtol=2e-4, atol=2e-4), t
    assert np.all(rows[[0, 3, 19, 40]] == 9.0)               # nothing else was written (slot -1 skipped)
    qn, qr = mixers.rope_split_q(proj.to(device), inv.to(device), pos.to(device), H, D, Dr, rot, interleaved=True, mag=mag,
                                 off=R + Dr)
    q = pn[:, R + Dr:R + Dr + H * (D + Dr)].reshape(T, H, D + Dr)
    assert close(qn, q[:, :, :D].transpose(1, 0, 2), 1e-6, 1e-6)
    assert close(qr, oracle.rotate_pairs(q[:, :, D:], pos.numpy(), np.asarray(f), mag, rot), 2e-4, 2e-4)
    o = torch.randn(H, T, 7, generator=g)
    got = mixers.head_gate(o.to(device), proj.to(device), P - 3 - H)
    want = o.double().numpy().transpose(1, 0, 2) * oracle.sigmoid(pn[:, P - 3 - H:P - 3])[:, :, None]
    assert close(got, want.reshape(T, H * 7), 1e-5, 1e-5)
    assert close(mixers.head_gate(o.to(device), None), o.double().numpy().transpose(1, 0, 2).reshape(T, H * 7), 1e-6, 1e-6)


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


def _attend(device, q, k, v, dist, window, scale, cuts, dtype=torch.float32, norms=None, eps=0.0):
    """q [T, H, D], k [T, G, D], v [T, G, Dv]: through rope_append (no rotation; per-head norms if given) and
    sliding_attention with the sigmoid weights, in portions `cuts` (a portion of one row after the first runs the
    decode form).  -> [T, H * Dv]."""
    from ai_agent_kubectl_amd.ops import mixers

    T, H, D = q.shape
    G, Dv = k.shape[1], v.shape[2]
    pg = Paged(G, D, Dv, [T], device, dtype)
    rows = torch.cat([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], dim=1).to(dtype).to(device)
    qn, kn = (norms[0].to(device), norms[1].to(device)) if norms else (None, None)
    dd = dist.float().contiguous().to(device)
    out, at = [], 0
    for c in cuts:
        pos = list(range(at, at + c))
        p = torch.tensor(pos, dtype=torch.int32, device=device)
        sl = pg.slots(0, pos)
        qq = mixers.rope_append(rows[at:at + c].contiguous(), None, 1.0, p, sl, pg.k, pg.v, H, G, D, Dv, 0, qn, kn, eps)
        decode = c == 1 and at > 0
        out.append(mixers.sliding_attention(qq, pg.k, pg.v, pg.tables.to(device), None if decode else _seq_meta([c], device), p, sl,
                                            None, 0, window, 0, scale, max_q=c, dist=dd))
        at += c
    return torch.cat(out)


def _dist(g, H):
    return torch.stack([torch.rand(H, generator=g) * 1.3 + 0.2, torch.rand(H, generator=g) * 1.9 + 0.1, torch.rand(H, generator=g) * 3 - 2.5])


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,G,D,Dv,window", [(4, 2, 16, 8, 8), (3, 1, 7, 9, 21), (2, 2, 12, 20, 1), (1, 1, 8, 8, 0), (6, 3, 40, 24, 33),
                                             (6, 2, 64, 128, 36), (20, 1, 4, 4, 5), (4, 4, 5, 3, 17), (12, 1, 16, 256, 9)])
def test_sigmoid_attention_windows_groups_and_head_norms(device, H, G, D, Dv, window):
    g = torch.Generator().manual_seed(H * 100 + D)
    T, eps = 70, 1e-3
    q, k, v = torch.randn(T, H, D, generator=g) * 2, torch.randn(T, G, D, generator=g) * 0.5 + 0.3, torch.randn(T, G, Dv, generator=g)
    dist = _dist(g, H)
    wq, wk = torch.rand(D, generator=g) + 0.5, torch.rand(D, generator=g) + 0.5
    qd, kd = oracle.rms_div(q.double().numpy(), eps) * wq.double().numpy(), oracle.rms_div(k.double().numpy(), eps) * wk.double().numpy()
    r1, r2, pb = dist.double().numpy()
    want = oracle.sigmoid_attention(qd, kd, v.double().numpy(), 0.3, r1, r2, pb, window).reshape(T, H * Dv)
    for cuts in ([T], [33] + [1] * 37, [2, 2, 14, 1, 17, 3, 30, 1]):
        assert close(_attend(device, q, k, v, dist, window, 0.3, cuts, norms=(wq, wk), eps=eps), want, 1e-4, 2e-5), cuts


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("decode", [False, True])
@pytest.mark.parametrize("key,seen", [(60 - 11, True), (60 - 12, False), (60, True), (0, False)])
def test_window_edges_one_weight_stands_out(device, decode, key, seen):
    """Window 12, query at position 60.  All weights are pushed towards 0 by the per-head offset but the one of a key
    whose score stands out; that key has a value of its own.  It carries the result when it is the last key inside the
    window (or the query's own), and is absent one position further out, in a prompt row as in a decoded row."""
    g = torch.Generator().manual_seed(key)
    T, D, Dv, qpos = 61, 8, 4, 60
    q, k, v = torch.randn(T, 1, D, generator=g) * 0.1, torch.randn(T, 1, D, generator=g) * 0.1, torch.randn(T, 1, Dv, generator=g)
    q[qpos, 0], k[key, 0] = 0.0, 0.0
    q[qpos, 0, 0], k[key, 0, 0] = 6.0, 6.0
    v[key, 0] = torch.tensor([100.0, -100.0, 50.0, 25.0])
    dist = torch.tensor([[0.5], [1.0], [-8.0]])
    out = _attend(device, q, k, v, dist, 12, 1.0, [qpos, 1] if decode else [T])[qpos].cpu()
    want = oracle.sigmoid_attention(q.double().numpy(), k.double().numpy(), v.double().numpy(), 1.0, [0.5], [1.0], [-8.0], 12)[qpos, 0]
    assert np.allclose(out.double().numpy(), want, rtol=1e-4, atol=1e-4)
    assert (abs(float(out[0]) - 100.0) < 1.0) == seen


@pytest.mark.parametrize("device", DEVICES)
def test_distance_bias_and_offset_per_head(device):
    """Equal scores everywhere: the weights then depend on the distance alone, through each head's own r1, r2, pb."""
    T, H = 40, 3
    q, k = torch.zeros(T, H, 4), torch.zeros(T, 1, 4)
    v = torch.eye(T)[:, None, :]                                  # the result lists the weights of the keys
    dist = torch.tensor([[0.0, 1.0, 2.5], [1.0, 0.5, 3.0], [0.3, -1.0, 2.0]])
    out = _attend(device, q, k, v, dist, 0, 1.0, [25] + [1] * 15).cpu().double().numpy().reshape(T, H, T)
    for h in range(H):
        r1, r2, pb = [float(dist[i, h]) for i in range(3)]
        d = 39 - np.arange(T)
        assert np.allclose(out[39, h], oracle.sigmoid(pb - r1 * np.log(1 + r2 * d)), rtol=1e-4, atol=1e-6)
    # without a distance bias every key weighs the same, and the 40 weights sum to far more than 1: no softmax
    assert np.allclose(out[39, 0], oracle.sigmoid(0.3)) and out[39, 0].sum() > 20 and out[39, 2, 0] < 0.001 < out[39, 2, 39]


@pytest.mark.parametrize("device", DEVICES)
def test_far_key_among_hundreds_in_latent_attention(device):
    """450 positions over 29 scrambled pages, causal softmax over latent rows with interleaved rotation: the key at
    position 3 is the only one whose latent matches the last query's, and its latent comes back as the result."""
    from ai_agent_kubectl_amd.ops import mixers

    g = torch.Generator().manual_seed(5)
    T, H, R, Dr, key = 450, 2, 16, 8, 3
    proj = torch.randn(T, R + Dr, generator=g) * 0.3
    proj[key, :R] = 0.0
    proj[key, 5] = 3.0                                            # after the norm: one entry of size sqrt(R)
    pg = Paged(1, 1, 1, [T], device)
    cache = torch.zeros((pg.tables.max().item() + 1, BS, R + Dr), device=device)
    pos = torch.arange(T, dtype=torch.int32, device=device)
    sl = pg.slots(0, range(T))
    inv = torch.tensor(oracle.rotary_table(Dr, 100.0, None)[0], dtype=torch.float32, device=device)
    ones = torch.ones(R, device=device)
    q_lat = torch.randn(H, T, R, generator=g) * 0.3
    q_lat[:, T - 1] = 0.0
    q_lat[:, T - 1, 5] = 6.0
    q_rot = torch.randn(T, H, Dr, generator=g) * 0.3
    outs = []
    for cuts in ([T], [T - 1, 1]):
        at = 0
        for c in cuts:
            s = slice(at, at + c)
            mixers.latent_prep(proj[s].contiguous().to(device), 0, R, Dr, None, ones, inv, pos[s], sl[s], cache, Dr, 1e-6,
                               interleaved=True, mag=1.0)
            o = mixers.window_attention(q_lat[:, s].contiguous().to(device), q_rot[s].contiguous().to(device), cache, pg.tables.to(device),
                                        None if c == 1 else _seq_meta([c], device), pos[s], sl[s], None, 0, 1.0)
            at += c
        outs.append(o[:, -1].cpu())
    for o in outs:
        assert abs(float(o[0, 5]) - 4.0) < 0.05 and float(o[0].abs().sum()) < 4.5 and abs(float(o[1, 5]) - 4.0) < 0.05
    assert torch.allclose(outs[0], outs[1], atol=1e-4)


def _route_inputs(g, T, W, E):
    h, wr = torch.randn(T, W, generator=g), torch.randn(E, W, generator=g) * (1.5 * W ** -0.5)
    return h, wr


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("E,top", [(5, 2), (8, 1), (4, 4), (70, 3)])
def test_sigmoid_router(device, E, top):
    from ai_agent_kubectl_amd.ops import mixers

    g = torch.Generator().manual_seed(E)
    h, wr = _route_inputs(g, 11, 32, E)
    ids, w = mixers.moe_route(h.to(device), wr.to(device), None, top, 1, 1, sigmoid=True, renorm=False)
    wi, ww = oracle.route(h.double().numpy(), {"router": wr.double().numpy()}, "", top)
    assert np.array_equal(ids.cpu().numpy(), wi) and np.allclose(w.cpu().numpy(), ww, rtol=1e-5, atol=1e-6)
    assert ww.sum(-1).max() > 1.05 or top == 1               # sigmoid scores, not renormalised: they need not sum to 1
    ids2, w2 = mixers.moe_route(h.to(device), wr.to(device), None, top, 1, 1, sigmoid=True, renorm=True)
    assert np.allclose(w2.cpu().numpy().sum(-1), 1.0, atol=1e-5) and np.array_equal(ids2.cpu().numpy(), wi)


def _experts_oracle(h, w_gu, w_dn, ids, w):
    T, ff = h.shape[0], w_dn.shape[2]
    out = np.zeros((T, h.shape[1]))
    for t in range(T):
        for e, s in zip(ids[t], w[t]):
            x = s * h[t]
            out[t] += w_dn[e] @ (oracle.silu(w_gu[e, :ff] @ x) * (w_gu[e, ff:] @ x))
    return out


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("T", [3, 40, 300])
def test_experts_with_scaled_inputs(device, T):
    """The score multiplies the expert's input, ahead of its nonlinearity; three step sizes take the three paths
    (matrix-vector kernels, sorted rows with one product pair per expert)."""
    from ai_agent_kubectl_amd.ops import mixers

    g = torch.Generator().manual_seed(T)
    W, ff, E, top = 24, 10, 5, 2
    h = torch.randn(T, W, generator=g)
    w_gu, w_dn = torch.randn(E, 2 * ff, W, generator=g) * W ** -0.5, torch.randn(E, W, ff, generator=g) * ff ** -0.5
    ids = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(T)]).to(torch.int32)
    w = torch.rand(T, top, generator=g) * 1.5 + 0.1
    want = _experts_oracle(h.double().numpy(), w_gu.double().numpy(), w_dn.double().numpy(), ids.numpy(), w.double().numpy())
    got = mixers.moe_experts(h.to(device), w_gu.to(device), w_dn.to(device), ids.to(device), w.to(device), scale_input=True)
    assert close(got, want, 1e-4, 1e-5)
    outside = mixers.moe_experts(h.to(device), w_gu.to(device), w_dn.to(device), ids.to(device), w.to(device))
    assert not close(outside, want, 1e-2, 1e-2)               # weighting the output is another function


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
@pytest.mark.parametrize("name", ["base", "odd"])
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
def test_shared_layers_have_caches_of_their_own(tmp_path, device):
    """A layer that runs on another's tensors sees other inputs, so its cache differs; with the owner's cache or
    with weights of its own the logits would differ from the oracle's."""
    c, W, path = model_for(tmp_path, "base", seed=4)
    sess = session(path, device)
    model = sess.runner.model
    assert model.layers[4] is model.layers[2] and len({id(k) for k in sess.runner.k_cache}) == 5
    toks = tokens_for(c, 30, seed=5)
    assert rel_err(replay(sess, toks, [20] + [1] * 10, end=False), want_logits(c, W, toks)) < tol("float32")
    assert not torch.equal(sess.runner.k_cache[2], sess.runner.k_cache[4])
    own = dict(c, layers=[dict(L) for L in c["layers"]])
    del own["layers"][4]["weights_of"]
    assert rel_err(want_logits(own, oracle.random_tensors(own, 4), toks), want_logits(c, W, toks)) > 1e-2


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", VARIANTS)
def test_decode_token_by_token(tmp_path, device, name):
    """10 prompt tokens, then 60 decoded one by one: over page borders and past every window."""
    c, W, path = model_for(tmp_path, name, seed=3)
    toks = tokens_for(c, 70, seed=4)
    sess = session(path, device)
    assert rel_err(replay(sess, toks, [10] + [1] * 60), want_logits(c, W, toks)) < tol("float32")


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name,cuts", [("base", [2, 2, 3, 9, 2, 16, 1, 1, 15, 2]), ("odd", [5, 5, 2, 11, 17, 13]),
                                       ("window_one", [1, 2, 2, 2, 2, 2, 30, 2, 10]), ("no_mask", [16, 16, 2, 14, 5])])
def test_portions(tmp_path, device, name, cuts):
    c, W, path = model_for(tmp_path, name, seed=5)
    toks = tokens_for(c, sum(cuts), seed=6)
    sess = session(path, device)
    assert rel_err(replay(sess, toks, cuts), want_logits(c, W, toks)) < tol("float32")


@pytest.mark.parametrize("device", DEVICES)
def test_mixed_batches_and_pages_reused(tmp_path, device):
    """Six unequal requests through a pool of 112 tokens: portions of some beside single tokens of others; a
    finished request's pages go to the next one, and what they held must not show."""
    c, W, path = model_for(tmp_path, "base", seed=4)
    sess = session(path, device, max_tokens=112, max_requests=3)
    lens = {"a": 40, "b": 9, "c": 33, "d": 21, "e": 30, "f": 17}
    toks = {k: tokens_for(c, n, seed=10 + i) for i, (k, n) in enumerate(lens.items())}
    plan = [[("a", 7)], [("a", 2), ("b", 3)], [("a", 1), ("b", 1), ("c", 20)], [("a", 14), ("b", 1), ("c", 2)],
            [("b", 4), ("c", 1), ("a", 1)], [("c", 10), ("a", 15)], [("d", 21)], [("e", 2)],
            [("e", 27), ("f", 16)], [("e", 1), ("f", 1)]]
    got = run_plan(sess, toks, plan)
    assert sess.sched.bm.num_free == sess.sched.bm.num_blocks
    for k in lens:
        assert rel_err(got[k], want_logits(c, W, toks[k])) < tol("float32"), k


@pytest.mark.parametrize("device", DEVICES)
def test_batch_against_each_alone(tmp_path, device):
    """Three unequal requests decoded together give what each gives alone, to rounding."""
    c, W, path = model_for(tmp_path, "odd", seed=7)
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
    """A 150-position window and causal latent attention over a 400-token sequence, the last 230 decoded one by one."""
    c = make_config([attention_layer(heads=2, kv_heads=1, dim=8, vdim=8, window=150, ff=12),
                     latent_layer(heads=2, dim=4, rot_dim=8, vdim=4, kv_rank=8, scaling=(8.0, 128, 16.0, 1.0), mlp=None)], width=16, vocab=64)
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
@pytest.mark.parametrize("prefix", [False, True])
def test_generate_greedy_through_scheduler(tmp_path, device, prefix):
    """Greedy generation through build_engine / generate_blocking: the scheduler chunks the prompts (12 tokens a
    step) and batches at most three requests; with prefix caching, prompts that share their first 32 tokens reuse
    the pages of the first."""
    from ai_agent_kubectl_amd.engine.builder import EngineOptions, build_engine
    from ai_agent_kubectl_amd.engine.sequence import SamplingParams

    c, W, path = model_for(tmp_path, "base", seed=6)
    head = tokens_for(c, 32, seed=19)
    prompts = [(head if prefix else []) + tokens_for(c, n, seed=20 + n) for n in (5, 19, 1, 26, 8, 13)]
    eng = build_engine(EngineOptions(model=path, device=device, dtype="float32", max_batch=3, max_batched_tokens=12,
                                     max_model_len=96, kv_cache_tokens=384, graph_buckets=(1, 2, 3), use_graphs=False,
                                     safe_decode=False, ignore_eos=True, prefix_caching=prefix))
    assert eng.bm.prefix_caching == prefix
    seqs = eng.generate_blocking(prompts, SamplingParams(max_new_tokens=10, ignore_eos=True, safe_decode=False))
    for p, s in zip(prompts, seqs):
        toks = list(p)
        for _ in range(10):
            toks.append(int(np.argmax(want_logits(c, W, toks)[-1])))
        assert s.generated == toks[len(p):]


def test_config_reader(tmp_path):
    from ai_agent_kubectl_amd.models.config import ZibinexConfig, get_config

    for name in VARIANTS:
        c, W, path = model_for(tmp_path, name)
        cfg = get_config(path)
        assert cfg.family == "zibinex" and cfg.num_layers == len(c["layers"]) and not cfg.has_state
        assert ZibinexConfig.from_dict(cfg.to_dict(), cfg.name) == cfg
    cfg = get_config(model_for(tmp_path, "no_mask")[2])
    assert cfg.layers[0].mixer.window == 0 and cfg.layers[1].mixer.rot.dims == 0 and cfg.layers[1].mlp is None
    assert cfg.layers[2].mixer.window == 5 and cfg.layers[2].mixer.rot.factor == 16.0
    cfg = get_config(model_for(tmp_path, "odd")[2])
    assert cfg.owner(0) == 2 and cfg.owner(2) == 2 and cfg.norm_eps == 1e-3
    assert cfg.kv_bytes_per_token(4) == 4 * (2 * (7 + 9) + 11 + 6)
    for edit in (lambda b: b["layers"][0].__setitem__("type", "convolution"),
                 lambda b: b["layers"][1]["mixer"].__setitem__("kv_heads", 3),       # 4 heads in groups of 3
                 lambda b: b["layers"][1]["mlp"].__setitem__("kind", "experts"),
                 lambda b: b["layers"][1]["mlp"]["router"].__setitem__("top", 9),     # more than there are experts
                 lambda b: b["layers"][4].__setitem__("weights_of", 1),               # another kind of layer
                 lambda b: b["layers"][4]["mixer"].__setitem__("kv_rank", 10),        # other tensor sizes than its owner's
                 lambda b: b["layers"][4].__setitem__("weights_of", 4),               # itself
                 lambda b: b["layers"][2].__setitem__("weights_of", 4)):              # a layer that has none of its own
        bad = variant("base")
        edit(bad)
        with pytest.raises(ValueError):
            ZibinexConfig.from_dict(bad)
    assert get_config("tiny-zibinex").layers[4].weights_of == 2


def test_loader_checks_shapes(tmp_path):
    from ai_agent_kubectl_amd.models.config import get_config
    from ai_agent_kubectl_amd.models.weights import ParallelInfo, build_weights, zibinex_columns, zibinex_random_weights

    c, W, path = model_for(tmp_path, "base")
    Wl = build_weights(path, get_config(path), ParallelInfo(), dtype=torch.float32)
    assert "layers.4.wo" not in Wl and Wl["lm_head"] is Wl["embed"]
    assert torch.allclose(Wl["layers.0.norm1"], 1.0 + W["l0.norm1"]) and Wl["layers.1.dist"].shape == (3, 4)
    W2 = dict(W)
    W2["l1.mix.k.b"] = W["l1.mix.k.b"][:-1]
    bad = write_checkpoint(tmp_path / "bad", c, W2)
    with pytest.raises((ValueError, RuntimeError)):
        build_weights(bad, get_config(bad), ParallelInfo(), dtype=torch.float32)
    del W2["l1.mix.k.b"]
    bad = write_checkpoint(tmp_path / "bad2", c, W2)
    with pytest.raises(KeyError):
        build_weights(bad, get_config(bad), ParallelInfo(), dtype=torch.float32)
    cfg = get_config("tiny-zibinex")
    Wr = zibinex_random_weights(cfg, seed=1, dtype=torch.float32)
    col = zibinex_columns(cfg.layers[0].mixer)
    assert col == {"kv": 0, "q": 48, "g": 48 + 4 * 32, "total": 184} and Wr["layers.0.w_in"].shape == (184, 128)
    assert Wr["layers.2.w_gu_e"].shape == (6, 128, 128)


# ---------------------------------------------------------------------------------------------------
# GPU only: the bf16 engine, wider shapes (the matrix-core kernels), captured decode
@pytest.mark.gpu
@pytest.mark.parametrize("name", ["base", "odd"])
def test_bf16_engine(tmp_path, name):
    c, W, path = model_for(tmp_path, name, seed=12, every_expert=True)
    toks = tokens_for(c, 60, seed=13)
    want = want_logits(c, W, toks)
    sess = session(path, "cuda", dtype="bfloat16")
    assert ok_bf16(replay(sess, toks, [60]), want)
    assert ok_bf16(replay(sess, toks, [7, 2, 20, 1, 1, 1, 12, 16], rid="p"), want)


def wide_config():
    """Head sizes the matrix-core kernels take: latent rows of 64 + 32 entries, key / value heads of 128 / 64 with 4
    query heads each, expert and dense widths that are multiples of 32."""
    return make_config([latent_layer(heads=4, dim=32, rot_dim=32, vdim=48, kv_rank=64, base=10000.0, scaling=(8.0, 256, 32.0, 1.0),
                                     scale=0.125, mlp="dense", ff=256, limit=1.0),
                        attention_layer(heads=8, kv_heads=2, dim=128, vdim=64, window=40, scale=0.09, ff=96, experts=6, top=2),
                        shared(latent_layer(heads=4, dim=32, rot_dim=32, vdim=48, kv_rank=64, base=10000.0, scaling=(8.0, 256, 32.0, 1.0),
                                            scale=0.125, mlp="dense", ff=256, limit=1.0), 0),
                        attention_layer(heads=2, kv_heads=2, dim=64, vdim=128, window=0, scale=0.12, mlp=None)], width=256, vocab=512)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_wider_shapes_gpu(tmp_path, dtype):
    c = wide_config() if dtype == "float32" else all_experts(wide_config())
    W = oracle.random_tensors(c, 14)
    path = write_checkpoint(tmp_path / "wide", c, W)
    toks = tokens_for(c, 100, seed=15)
    want = want_logits(c, W, toks)
    sess = session(path, "cuda", dtype=dtype)
    for rid, cuts in (("p", [64, 2, 1, 1, 30, 1, 1]), ("w", [100])):
        got = replay(sess, toks, cuts, rid=rid)
        assert rel_err(got, want) < tol(dtype) if dtype == "float32" else ok_bf16(got, want), cuts


@pytest.mark.gpu
def test_mixed_steps_on_the_matrix_cores(tmp_path):
    """bf16 engine at the wide sizes: single decoded rows of two requests ahead of a prompt portion of a third in one
    step (single rows and portions take different forms of the attention kernels), then the roles change."""
    c = all_experts(wide_config())
    W = oracle.random_tensors(c, 21)
    path = write_checkpoint(tmp_path / "mixed", c, W)
    toks = {k: tokens_for(c, n, seed=50 + n) for k, n in (("a", 44), ("b", 37), ("c", 90))}
    sess = session(path, "cuda", dtype="bfloat16", max_tokens=256)
    plan = [[("a", 40), ("b", 35)], [("a", 1), ("b", 1), ("c", 50)], [("a", 1), ("c", 1), ("b", 1)], [("c", 37), ("a", 1)],
            [("c", 1), ("a", 1)], [("c", 1)]]
    got = run_plan(sess, toks, plan)
    for k in toks:
        assert ok_bf16(got[k], want_logits(c, W, toks[k])), k


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
@pytest.mark.parametrize("H,G,D,Dv,window", [(4, 1, 64, 64, 44), (6, 2, 64, 128, 36), (8, 2, 128, 128, 100), (2, 2, 128, 64, 0),
                                             (8, 1, 256, 256, 17), (4, 4, 64, 256, 1), (3, 1, 128, 128, 16)])
def test_sigmoid_attention_matrix_core_kernel(H, G, D, Dv, window):
    """bf16 rows run on the matrix cores: against the oracle on the bf16-rounded inputs, whole, in portions whose rows
    start anywhere in a page and row by row; the vector kernel agrees."""
    from ai_agent_kubectl_amd.ops import mixers

    g = torch.Generator().manual_seed(H + D + window)
    T = 150
    bf = lambda t: t.to(torch.bfloat16).float()
    q, k, v = bf(torch.randn(T, H, D, generator=g)), bf(torch.randn(T, G, D, generator=g)), bf(torch.randn(T, G, Dv, generator=g))
    dist = _dist(g, H)
    r1, r2, pb = dist.double().numpy()
    scale = D ** -0.5 * 2
    want = oracle.sigmoid_attention(q.double().numpy(), k.double().numpy(), v.double().numpy(), scale, r1, r2, pb, window).reshape(T, H * Dv)
    assert mixers.require_mixers().ka_sliding_attention_tile_ok(H, G, D, Dv, BS)
    outs = []
    for tile in (True, False):
        mixers.SLIDING_TILE = tile
        try:
            for cuts in ([T], [37, 9, 70, 1, 33], [16, 16, 8, 100] + [1] * 10):
                got = _attend("cuda", q, k, v, dist, window, scale, cuts, dtype=torch.bfloat16)
                assert close(got, want, 2e-2, 3e-2), (tile, cuts)
                outs.append(got.float().cpu())
        finally:
            mixers.SLIDING_TILE = True
    assert torch.allclose(outs[0], outs[3], rtol=1e-2, atol=3e-2)     # the two kernels: a bf16 rounding of the unnormalised sums apart


@pytest.mark.gpu
@pytest.mark.parametrize("decode", [False, True])
@pytest.mark.parametrize("key,seen", [(140 - 43, True), (140 - 44, False), (140, True), (0, False)])
def test_window_edges_on_the_matrix_cores(decode, key, seen):
    """Window 44, the query at position 140 (a row of a 150-row portion, or a single row; bf16, head size 64): the key
    whose weight stands out carries the result exactly when the mask lets it."""
    g = torch.Generator().manual_seed(key)
    T, D, Dv, qpos = 150, 64, 64, 140
    q, k, v = torch.randn(T, 2, D, generator=g) * 0.05, torch.randn(T, 1, D, generator=g) * 0.05, torch.randn(T, 1, Dv, generator=g)
    q[qpos], k[key] = 0.0, 0.0
    q[qpos, :, 0], k[key, 0, 0] = 6.0, 6.0
    v[key, 0] = 100.0
    dist = torch.tensor([[0.5, 0.25], [1.0, 2.0], [-8.0, -9.0]])
    cuts = [qpos, 1] + [9] if decode else [T]
    out = _attend("cuda", q, k, v, dist, 44, 1.0, cuts, dtype=torch.bfloat16)[qpos].float().cpu()
    assert (abs(float(out[0]) - 100.0) < 2.0) == seen and (abs(float(out[Dv]) - 100.0) < 2.0) == seen


@pytest.mark.gpu
@pytest.mark.parametrize("T", [5, 200, 1500])
def test_experts_with_scaled_inputs_bf16(T):
    """bf16 steps: rows grouped by expert on the matrix cores (up to 1024 rows), sorted rows beyond."""
    from ai_agent_kubectl_amd.ops import mixers

    g = torch.Generator().manual_seed(T)
    W, ff, E, top = 64, 32, 6, 3
    bf = lambda t: t.to(torch.bfloat16)
    h = bf(torch.randn(T, W, generator=g))
    w_gu, w_dn = bf(torch.randn(E, 2 * ff, W, generator=g) * W ** -0.5), bf(torch.randn(E, W, ff, generator=g) * ff ** -0.5)
    ids = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(T)]).to(torch.int32)
    w = torch.rand(T, top, generator=g) * 1.5 + 0.1
    want = _experts_oracle(h.double().numpy(), w_gu.double().numpy(), w_dn.double().numpy(), ids.numpy(), w.double().numpy())
    got = mixers.moe_experts(h.cuda(), w_gu.cuda(), w_dn.cuda(), ids.cuda(), w.cuda(), scale_input=True)
    assert close(got, want, 3e-2, 3e-2)
