"""A plain, slow restatement of the Nizorax design in float64 PyTorch, one function per mechanism.

Nothing here is shared with the product (which is C++ / HIP behind the C ABI): the tests build small random models, write them as a
config.json + model.safetensors folder, run them through the engine and compare with these functions.

The design: a residual stream x [T, W]; every layer does x += LN_b(mixer(C(LN(x)))) and then x += LN_b'(ff(C'(LN'(x)))), with LN a layer norm
with weight and bias and C(h) = h + a short causal convolution of h over time, per channel.  Mixers: `attention` (grouped-query, rotated keys,
sliding window, two score maps per head combined as a difference) and `lightning` (linear attention with a decaying state).  Feed-forward: dense
with a polynomial activation whose terms are unit-normed, or a mixture of gated experts chosen by sigmoid scores within the best groups.
A span of layers can run several times in a row with the same weights.

Notation: T tokens, W width, H heads, G key/value heads, dn the size of a query / key map, dv the value size of a head.
A model is (config dict, {tensor name: float64 tensor}).
"""
import json
import math
import os
import struct

import numpy as np
import torch

F = torch.float64


# ---------------------------------------------------------------------------------------------------------------- pieces
def unit_rms(x, eps):
    """x over the root of (its mean square + eps), along the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def layer_norm(x, w, b, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def conv_added(h, w, history=None):
    """h + conv(h): out_t = h_t + sum_j w[:, j] h_(t - taps + 1 + j); `history` [taps - 1, W] are the inputs before h (zeros at a sequence's start).
    -> (out, the last taps - 1 inputs)."""
    taps = w.shape[1]
    T, W = h.shape
    hist = torch.zeros(taps - 1, W, dtype=F) if history is None else history
    full = torch.cat([hist, h], 0)
    out = h.clone()
    for t in range(T):
        for j in range(taps):
            out[t] = out[t] + w[:, j] * full[t + j]
    return out, full[full.shape[0] - (taps - 1):]


def rotary_frequencies(rot):
    """f_i = base^(-2i/dims), then by wavelength l = 2 pi / f: short waves stay, long waves are slowed by `factor`, a blend between."""
    d = int(rot["dims"])
    f = [float(rot["base"]) ** (-2.0 * i / d) for i in range(d // 2)]
    sc = rot.get("scaling")
    if sc:
        out = []
        for fi in f:
            l = 2.0 * math.pi / fi
            if l < sc["original"] / sc["high"]:
                out.append(fi)
            elif l > sc["original"] / sc["low"]:
                out.append(fi / sc["factor"])
            else:
                s = (sc["original"] / l - sc["low"]) / (sc["high"] - sc["low"])
                out.append((1.0 - s) * fi / sc["factor"] + s * fi)
        f = out
    return torch.tensor(f, dtype=F)


def rotate_pairs(x, pos, rot):
    """x [T, n, dn]: entries (2i, 2i+1), i < dims/2, of every vector turn by pos * f_i; the rest pass."""
    d = int(rot["dims"])
    if d == 0:
        return x
    ang = pos.to(F)[:, None] * rotary_frequencies(rot)[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    u, v = x[..., 0:d:2], x[..., 1:d:2]
    y = x.clone()
    y[..., 0:d:2] = u * c - v * s
    y[..., 1:d:2] = v * c + u * s
    return y


def visible(qpos, kpos, window):
    """[Tq, Tk] bool: key j is seen from i iff 0 <= i - j < window (window None or 0: every earlier key)."""
    d = qpos[:, None] - kpos[None, :]
    ok = d >= 0
    if window:
        ok = ok & (d < window)
    return ok


def lambda_of(w, pre, diff):
    return float(torch.exp((w[pre + "lq1"] * w[pre + "lk1"]).sum()) - torch.exp((w[pre + "lq2"] * w[pre + "lk2"]).sum()) + diff)


def diff_attention(h, w, pre, mx, eps, pos=None, past=None):
    """h [T, W] at positions pos; past = (keys [P, G, 2, dn] rotated, values [P, G, dv], their positions) from earlier tokens.
    -> (out [T, W], (keys, values, positions) including this call's)."""
    T = h.shape[0]
    H, G, dn, dv = mx["heads"], mx.get("kv_heads", mx["heads"]), mx["dim"], mx["vdim"]
    pos = torch.arange(T) if pos is None else pos
    q = (h @ w[pre + "q"].T).view(T, H * 2, dn)
    k = (h @ w[pre + "k"].T).view(T, G * 2, dn)
    v = (h @ w[pre + "v"].T).view(T, G, dv)
    q = rotate_pairs(q, pos, mx["rot"]).view(T, H, 2, dn)
    k = rotate_pairs(k, pos, mx["rot"]).view(T, G, 2, dn)
    kpos = pos
    if past is not None:
        k, v, kpos = torch.cat([past[0], k]), torch.cat([past[1], v]), torch.cat([past[2], pos])
    lam = lambda_of(w, pre, mx["diff"])
    ok = visible(pos, kpos, mx.get("mask", {}).get("size"))
    out = torch.zeros(T, H, dv, dtype=F)
    for hh in range(H):
        g = hh // (H // G)
        maps = []
        for m in range(2):
            s = (q[:, hh, m] @ k[:, g, m].T) * mx["scale"]
            s = s.masked_fill(~ok, -math.inf)
            maps.append(torch.softmax(s, -1) @ v[:, g])
        o = maps[0] - lam * maps[1]
        out[:, hh] = unit_rms(o, eps) * (1.0 - mx["diff"])
    return out.reshape(T, H * dv) @ w[pre + "o"].T, (k, v, kpos)


def silu(z):
    return z * torch.sigmoid(z)


def lightning(h, w, pre, mx, eps, state=None):
    """The recurrence token by token.  state [H, dn, dv] or None (zeros).  -> (out [T, W], state)."""
    T = h.shape[0]
    H, dn, dv = mx["heads"], mx["dim"], mx["vdim"]
    dec = mx["decay"] if isinstance(mx["decay"], (list, tuple)) else [mx["decay"]] * H
    q = silu(h @ w[pre + "q"].T).view(T, H, dn)
    k = silu(h @ w[pre + "k"].T).view(T, H, dn)
    v = silu(h @ w[pre + "v"].T).view(T, H, dv)
    S = torch.zeros(H, dn, dv, dtype=F) if state is None else state.clone()
    o = torch.zeros(T, H, dv, dtype=F)
    for t in range(T):
        for hh in range(H):
            S[hh] = dec[hh] * S[hh] + torch.outer(k[t, hh], v[t, hh])
            o[t, hh] = S[hh].T @ q[t, hh]
    y = unit_rms(o.reshape(T, H * dv), eps) * w[pre + "norm"] * torch.sigmoid(h @ w[pre + "g"].T)
    return y @ w[pre + "o"].T, S


def polynorm(z, coef, eps):
    a, b, c, e = [float(x) for x in coef]
    return a * unit_rms(z, eps) + b * unit_rms(z ** 2, eps) + c * unit_rms(z ** 3, eps) + e


def dense_ff(h, w, pre, eps):
    return polynorm(h @ w[pre + "up"].T, w[pre + "act"], eps) @ w[pre + "down"].T


def gated_expert(h, w, pre):
    return (silu(h @ w[pre + "gate"].T) * (h @ w[pre + "up"].T)) @ w[pre + "down"].T


def route(h, w_router, rt):
    """-> (ids [T, top], weights [T, top]): sigmoid scores; the groups with the largest sum of their two best scores stay open; the `top` best
    open experts, weighted by score * scale."""
    s = torch.sigmoid(h @ w_router.T)
    T, E = s.shape
    top, gr = rt["top"], rt.get("groups")
    ids, wts = [], []
    for t in range(T):
        allowed = torch.ones(E, dtype=torch.bool)
        if gr and gr["count"] > 1:
            per = E // gr["count"]
            gs = torch.stack([torch.sort(s[t, g * per:(g + 1) * per], descending=True).values[:2].sum() for g in range(gr["count"])])
            keep = torch.sort(gs, descending=True, stable=True).indices[:gr["keep"]]
            allowed[:] = False
            for g in keep.tolist():
                allowed[g * per:(g + 1) * per] = True
        sc = torch.where(allowed, s[t], torch.full_like(s[t], -1.0))
        pick = torch.sort(sc, descending=True, stable=True).indices[:top]
        ids.append(pick)
        wts.append(s[t, pick] * rt.get("scale", 1.0))
    return torch.stack(ids), torch.stack(wts)


def mixture(h, w, pre, ml):
    ids, wts = route(h, w[pre + "router"], ml["router"])
    out = torch.zeros(h.shape[0], w[pre + "e0.down"].shape[0], dtype=F)
    for t in range(h.shape[0]):
        for e, a in zip(ids[t].tolist(), wts[t]):
            out[t] = out[t] + a * gated_expert(h[t:t + 1], w, "%se%d." % (pre, e))[0]
    if ml.get("shared"):
        out = out + gated_expert(h, w, pre + "shared.")
    return out


# ---------------------------------------------------------------------------------------------------------------- the model
def layer_runs(cfg):
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp:
        return list(range(n))
    return list(range(lp["start"])) + list(range(lp["start"], lp["stop"])) * lp["times"] + list(range(lp["stop"], n))


def forward(cfg, w, tokens, return_layers=False):
    """Logits [T, vocab] of a whole sequence (and the stream after every layer run)."""
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.tensor(list(tokens))] * cfg["embedding"]["scale"]
    streams = []
    for i in layer_runs(cfg):
        L, p = cfg["layers"][i], "l%d." % i
        h, _ = conv_added(layer_norm(x, w[p + "norm1"], w[p + "norm1.b"], eps), w[p + "canon1"])
        if L["type"] == "attention":
            y, _ = diff_attention(h, w, p + "mix.", L["mixer"], eps)
        else:
            y, _ = lightning(h, w, p + "mix.", L["mixer"], eps)
        x = x + layer_norm(y, w[p + "norm1b"], w[p + "norm1b.b"], eps)
        ml = L.get("mlp")
        if ml:
            h, _ = conv_added(layer_norm(x, w[p + "norm2"], w[p + "norm2.b"], eps), w[p + "canon2"])
            y = dense_ff(h, w, p + "mlp.", eps) if ml["kind"] == "dense" else mixture(h, w, p + "mlp.", ml)
            x = x + layer_norm(y, w[p + "norm2b"], w[p + "norm2b.b"], eps)
        streams.append(x)
    logits = layer_norm(x, w["final.norm"], w["final.norm.b"], eps) @ w["head"].T * cfg["logit_scale"]
    return (logits, torch.stack(streams)) if return_layers else logits


def closest_call(cfg, w, tokens):
    """The smallest gap, over all positions and mixture layers, between a score (or group score) that was taken and the best one that was not:
    a model and tokens whose gap is wide give the same choice of experts under bfloat16 rounding."""
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.tensor(list(tokens))] * cfg["embedding"]["scale"]
    gap = math.inf
    for i in layer_runs(cfg):
        L, p = cfg["layers"][i], "l%d." % i
        h, _ = conv_added(layer_norm(x, w[p + "norm1"], w[p + "norm1.b"], eps), w[p + "canon1"])
        y = diff_attention(h, w, p + "mix.", L["mixer"], eps)[0] if L["type"] == "attention" else lightning(h, w, p + "mix.", L["mixer"], eps)[0]
        x = x + layer_norm(y, w[p + "norm1b"], w[p + "norm1b.b"], eps)
        ml = L.get("mlp")
        if not ml:
            continue
        h, _ = conv_added(layer_norm(x, w[p + "norm2"], w[p + "norm2.b"], eps), w[p + "canon2"])
        if ml["kind"] == "moe":
            rt = ml["router"]
            s = torch.sigmoid(h @ w[p + "mlp.router"].T)
            E, gr = s.shape[1], rt.get("groups")
            for t in range(s.shape[0]):
                allowed = torch.ones(E, dtype=torch.bool)
                if gr and gr["count"] > 1:
                    per = E // gr["count"]
                    gs = torch.sort(torch.stack([torch.sort(s[t, g * per:(g + 1) * per], descending=True).values[:2].sum() for g in range(gr["count"])]),
                                    descending=True)
                    if gr["keep"] < gr["count"]:
                        gap = min(gap, float(gs.values[gr["keep"] - 1] - gs.values[gr["keep"]]))
                    allowed[:] = False
                    for g in gs.indices[:gr["keep"]].tolist():
                        allowed[g * per:(g + 1) * per] = True
                sc = torch.sort(s[t][allowed], descending=True).values
                if rt["top"] < sc.numel():
                    gap = min(gap, float(sc[rt["top"] - 1] - sc[rt["top"]]))
        y = dense_ff(h, w, p + "mlp.", eps) if ml["kind"] == "dense" else mixture(h, w, p + "mlp.", ml)
        x = x + layer_norm(y, w[p + "norm2b"], w[p + "norm2b.b"], eps)
    return gap


def greedy(cfg, w, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(torch.argmax(forward(cfg, w, toks)[-1])))
    return toks[len(prompt):]


# ------------------------------------------------------------------------------------------------------- files and makers
def bf16_round(t):
    return t.to(torch.float32).to(torch.bfloat16).to(F)


def tensor_shapes(cfg):
    W, V, taps = int(cfg["width"]), int(cfg["vocab"]), int(cfg["canon"]["taps"])
    s = {"embed": (V, W), "final.norm": (W,), "final.norm.b": (W,), "head": (V, W)}
    for i, L in enumerate(cfg["layers"]):
        p, mx, ml = "l%d." % i, L["mixer"], L.get("mlp")
        for nm in ("norm1", "norm1b") + (("norm2", "norm2b") if ml else ()):
            s[p + nm], s[p + nm + ".b"] = (W,), (W,)
        s[p + "canon1"] = (W, taps)
        if ml:
            s[p + "canon2"] = (W, taps)
        H, dn, dv = mx["heads"], mx["dim"], mx["vdim"]
        if L["type"] == "attention":
            G = mx.get("kv_heads", H)
            s[p + "mix.q"], s[p + "mix.k"], s[p + "mix.v"], s[p + "mix.o"] = (H * 2 * dn, W), (G * 2 * dn, W), (G * dv, W), (W, H * dv)
            for nm in ("lq1", "lk1", "lq2", "lk2"):
                s[p + "mix." + nm] = (dn,)
        else:
            s[p + "mix.q"], s[p + "mix.k"], s[p + "mix.v"], s[p + "mix.g"] = (H * dn, W), (H * dn, W), (H * dv, W), (H * dv, W)
            s[p + "mix.o"], s[p + "mix.norm"] = (W, H * dv), (H * dv,)
        if ml and ml["kind"] == "dense":
            s[p + "mlp.up"], s[p + "mlp.down"], s[p + "mlp.act"] = (ml["ff"], W), (W, ml["ff"]), (4,)
        elif ml:
            for e in range(ml["router"]["experts"]):
                q = "%smlp.e%d." % (p, e)
                s[q + "gate"], s[q + "up"], s[q + "down"] = (ml["expert"]["ff"], W), (ml["expert"]["ff"], W), (W, ml["expert"]["ff"])
            s[p + "mlp.router"] = (ml["router"]["experts"], W)
            if ml.get("shared"):
                sf = ml["shared"]["ff"]
                s[p + "mlp.shared.gate"], s[p + "mlp.shared.up"], s[p + "mlp.shared.down"] = (sf, W), (sf, W), (W, sf)
    return s


def random_weights(cfg, seed, gain=1.0):
    """bf16-representable random tensors: matrices ~ N(0, gain / fan_in), norm weights around one, biases and lambda vectors small."""
    g = torch.Generator().manual_seed(seed)
    w = {}
    for name, shp in tensor_shapes(cfg).items():
        leaf = name.split(".")[-1]
        if name.endswith(".act"):
            t = torch.tensor([0.9, 0.4, -0.3, 0.1], dtype=F) + 0.1 * torch.randn(4, generator=g, dtype=F)
        elif leaf in ("lq1", "lk1", "lq2", "lk2"):
            t = 0.3 * torch.randn(shp, generator=g, dtype=F)
        elif leaf.startswith("canon"):
            t = 0.4 * torch.randn(shp, generator=g, dtype=F)
        elif len(shp) == 1:
            t = 0.2 * torch.randn(shp, generator=g, dtype=F)
            if leaf != "b":
                t = t + 1.0
        elif name == "embed":
            t = torch.randn(shp, generator=g, dtype=F)
        elif leaf == "router":
            t = torch.randn(shp, generator=g, dtype=F) * math.sqrt(4.0 / shp[1])     # scores well apart: no close calls between experts
        else:
            t = torch.randn(shp, generator=g, dtype=F) * math.sqrt(gain / shp[1])
        w[name] = bf16_round(t)
    return w


def save_model(folder, cfg, w):
    """config.json + model.safetensors (bfloat16), written by hand: 8-byte length, JSON header, data."""
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    header, blobs, at = {}, [], 0
    for name, t in w.items():
        raw = t.to(torch.float32).to(torch.bfloat16).contiguous().view(torch.int16).numpy().tobytes()
        header[name] = {"dtype": "BF16", "shape": list(t.shape), "data_offsets": [at, at + len(raw)]}
        blobs.append(raw)
        at += len(raw)
    hj = json.dumps(header).encode()
    hj += b" " * (-len(hj) % 8)
    with open(os.path.join(folder, "model.safetensors"), "wb") as f:
        f.write(struct.pack("<Q", len(hj)))
        f.write(hj)
        for b in blobs:
            f.write(b)


def small_config(layers=("attention", "lightning"), mlps=("dense", "moe"), width=48, vocab=80, heads=4, kv_heads=2, dim=12, vdim=20, rot_dims=8,
                 window=9, diff=0.55, lheads=3, ldim=10, lvdim=14, decay=(0.5, 0.9, 0.99), ff=56, experts=6, top=2, groups=(3, 2), eff=16, shared_ff=24,
                 route_scale=1.7, taps=3, loop=None, scaling=True, eps=1e-5, base=10000.0, embed_scale=3.0, logit_scale=0.5):
    """A configuration whose sizes all differ from each other, so that a swapped pair shows.  mlps: one of "dense", "moe", None per layer."""
    ls = []
    for k, t in enumerate(layers):
        if t == "attention":
            rot = {"base": base * (1 + k), "dims": rot_dims}
            if scaling:
                rot["scaling"] = {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 32}
            mx = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "diff": diff, "scale": 1.0 / math.sqrt(dim), "mask": {"size": window}, "rot": rot}
        else:
            mx = {"heads": lheads, "dim": ldim, "vdim": lvdim, "decay": list(decay)[:lheads] if isinstance(decay, (list, tuple)) else decay}
        kind = mlps[k % len(mlps)]
        if kind == "dense":
            ml = {"kind": "dense", "ff": ff}
        elif kind == "moe":
            rt = {"experts": experts, "top": top, "scale": route_scale}
            if groups:
                rt["groups"] = {"count": groups[0], "keep": groups[1]}
            ml = {"kind": "moe", "expert": {"ff": eff}, "router": rt}
            if shared_ff:
                ml["shared"] = {"ff": shared_ff}
        else:
            ml = None
        ls.append({"type": t, "mixer": mx, "mlp": ml})
    cfg = {"architecture": "Nizorax", "layers": ls, "norm": {"eps": eps}, "canon": {"taps": taps}, "embedding": {"scale": embed_scale},
           "logit_scale": logit_scale, "vocab": vocab, "width": width}
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg
