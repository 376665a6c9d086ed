"""A plain, slow restatement of the Fabolorn design in float64 PyTorch, one function per mechanism.

Nothing here is shared with the product (which is C++ / HIP behind the C ABI): the tests build small random models, write them as a
config.json + model.safetensors folder, run them through the engine and compare with these functions.

Notation: W is the model width, T the number of tokens of a sequence, H heads, dn / dr the unrotated / rotated part of a query or key head,
dv the value size of a head, R the latent size.  A model is (config dict, {tensor name: float64 tensor}).
"""
import json
import math
import os
import struct

import numpy as np
import torch

F = torch.float64


# ---------------------------------------------------------------------------------------------------------------- pieces
def rms_unit(x, eps):
    """x over its root mean square, eps inside the root."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_around_zero(x, w, eps):
    """The layer / model norm: the stored weight is the distance from one."""
    return rms_unit(x, eps) * (1.0 + w)


def norm_plain(x, w, eps):
    return rms_unit(x, eps) * w


def rotary_frequencies(rot):
    """Per pair i: the angle step per position and the factor on cos and sin (1 without scaling)."""
    dims, base = int(rot["dims"]), float(rot["base"])
    i = torch.arange(dims // 2, dtype=F)
    f = base ** (-2.0 * i / dims)
    mag = 1.0
    sc = rot.get("scaling")
    if sc:
        factor, orig = float(sc["factor"]), float(sc["original"])

        def where(turns):
            return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
        lo = max(math.floor(where(float(sc["fast"]))), 0)
        hi = min(math.ceil(where(float(sc["slow"]))), dims - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        f = f / factor * ramp + f * (1.0 - ramp)
        mag = 0.1 * math.log(factor) + 1.0
    return f, mag


def rotate_pairs(x, pos, rot):
    """x [..., T, d]: the first rot.dims entries of the last axis in neighbouring pairs, the rest untouched.  pos [T]."""
    dims = int(rot["dims"])
    f, mag = rotary_frequencies(rot)
    a = pos.to(F)[:, None] * f[None, :]                    # [T, dims/2]
    c, s = torch.cos(a) * mag, torch.sin(a) * mag
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def visible(qpos, kpos, window):
    """[Tq, Tk] bool: the query at position i sees the key at position j.  window None: every j <= i; else the last `window` positions, itself
    included."""
    i = torch.as_tensor(qpos)[:, None]
    j = torch.as_tensor(kpos)[None, :]
    m = j <= i
    if window is not None:
        m = m & ((i - j) < window)
    return m


def attend(qn, qr, kn, kr, v, qpos, kpos, window, scale):
    """Softmax attention with a two-part score.  qn [Tq, H, dn], qr [Tq, H, dr] (rotated), kn [Tk, H, dn], kr [Tk, dr] (rotated, one for all heads),
    v [Tk, H, dv] -> [Tq, H, dv]."""
    s = (torch.einsum("thd,shd->hts", qn, kn) + torch.einsum("thd,sd->hts", qr, kr)) * scale
    s = s.masked_fill(~visible(qpos, kpos, window)[None], float("-inf"))
    return torch.einsum("hts,shd->thd", torch.softmax(s, dim=-1), v)


def latent_attention(h, w, pre, mx, eps, pos=None):
    """Both latent mixers.  h [T, W]; w: tensors; pre: '<layer>.mix.'; mx: the mixer's config.  With 'q_rank' in the config the query
    goes through a normed latent, otherwise one matrix; with 'mask' the keys are the last mask.size positions."""
    T = h.shape[0]
    H, dn, dr, dv, R = int(mx["heads"]), int(mx["dim"]), int(mx["rot_dim"]), int(mx["vdim"]), int(mx["kv_rank"])
    pos = torch.arange(T) if pos is None else pos
    if (pre + "dq") in w:
        q = norm_plain(h @ w[pre + "dq"].T, w[pre + "dq.norm"], eps) @ w[pre + "uq"].T
    else:
        q = h @ w[pre + "q"].T
    q = q.view(T, H, dn + dr)
    kv = h @ w[pre + "dkv"].T
    c = norm_plain(kv[:, :R], w[pre + "dkv.norm"], eps)     # [T, R]
    kr = rotate_pairs(kv[:, R:], pos, mx["rot"])            # [T, dr], one for all heads
    qr = rotate_pairs(q[:, :, dn:].transpose(0, 1), pos, mx["rot"]).transpose(0, 1)   # [T, H, dr]
    kn = (c @ w[pre + "uk"].T).view(T, H, dn)
    v = (c @ w[pre + "uv"].T).view(T, H, dv)
    window = int(mx["mask"]["size"]) if mx.get("mask") else None
    o = attend(q[:, :, :dn], qr, kn, kr, v, pos, pos, window, float(mx["scale"])).reshape(T, H * dv)
    o = o * torch.sigmoid(h @ w[pre + "g"].T)
    return o @ w[pre + "o"].T


def clipped_expert(h, w, pre, limit):
    g = (h @ w[pre + "gate"].T).clamp(max=limit)
    u = (h @ w[pre + "up"].T).clamp(-limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[pre + "down"].T


def route(h, w_router, top):
    """Chosen experts [T, top] and their weights: softmax over all experts, the chosen scores over their sum."""
    s = torch.softmax(h @ w_router.T, dim=-1)
    val, idx = torch.topk(s, top, dim=-1)
    return idx, val / (val.sum(-1, keepdim=True) + 1e-20)


def mixture(h, w, pre, ml):
    E, top = int(ml["router"]["experts"]), int(ml["router"]["top"])
    idx, wt = route(h, w[pre + "router"], top)
    out = torch.zeros(h.shape[0], w[pre + "e0.down"].shape[0], dtype=F)
    for e in range(E):
        y = clipped_expert(h, w, "%se%d." % (pre, e), float(ml["expert"]["limit"]))
        out += y * (wt * (idx == e)).sum(-1, keepdim=True)
    if ml.get("shared"):
        gate = torch.sigmoid(h @ w[pre + "shared.sg"].T)    # [T, 1]
        out += clipped_expert(h, w, pre + "shared.", float(ml["shared"]["limit"])) * gate
    return out


# ----------------------------------------------------------------------------------------------------------------- model
def layer_runs(cfg):
    """The layer index of every layer run, with a flag on the first layer of a repeated pass."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    runs = [(i, False) for i in range(a)]
    for _ in range(times):
        runs += [(i, i == a) for i in range(a, b)]
    return runs + [(i, False) for i in range(b, n)]


def forward(cfg, w, tokens, return_layers=False):
    """Logits [T, vocab] of one whole sequence (float64)."""
    eps = float(cfg["norm"]["eps"])
    x0 = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    x = x0
    seen = []
    for li, enters in layer_runs(cfg):
        L = cfg["layers"][li]
        if enters:
            x = torch.cat([x, x0], dim=-1) @ w["loop.in"].T
        pre = "l%d." % li
        if L["type"] not in ("latent_attention", "latent_attention_2"):
            raise ValueError(L["type"])
        y = latent_attention(norm_around_zero(x, w[pre + "norm1"], eps), w, pre + "mix.", L["mixer"], eps)
        if L.get("mlp"):
            y = y + mixture(norm_around_zero(x, w[pre + "norm2"], eps), w, pre + "mlp.", L["mlp"])
        x = x + y
        seen.append(x)
    logits = norm_around_zero(x, w["final.norm"], eps) @ w["head"].T
    return (logits, torch.stack(seen)) if return_layers else logits


# ------------------------------------------------------------------------------------------------------- files and makers
def bf16_round(t):
    """Round to bfloat16 and back (the stored precision of every weight)."""
    return t.to(torch.float32).to(torch.bfloat16).to(F)


def tensor_shapes(cfg):
    W, V = int(cfg["width"]), int(cfg["vocab"])
    s = {"embed": (V, W), "final.norm": (W,), "head": (V, W)}
    if cfg.get("loop"):
        s["loop.in"] = (W, 2 * W)
    for i, L in enumerate(cfg["layers"]):
        p, mx, ml = "l%d." % i, L["mixer"], L.get("mlp")
        H, dn, dr, dv, R = mx["heads"], mx["dim"], mx["rot_dim"], mx["vdim"], mx["kv_rank"]
        s[p + "norm1"] = (W,)
        if ml:
            s[p + "norm2"] = (W,)
        if L["type"] == "latent_attention":
            s[p + "mix.dq"] = (mx["q_rank"], W)
            s[p + "mix.dq.norm"] = (mx["q_rank"],)
            s[p + "mix.uq"] = (H * (dn + dr), mx["q_rank"])
        else:
            s[p + "mix.q"] = (H * (dn + dr), W)
        s[p + "mix.dkv"] = (R + dr, W)
        s[p + "mix.dkv.norm"] = (R,)
        s[p + "mix.uk"] = (H * dn, R)
        s[p + "mix.uv"] = (H * dv, R)
        s[p + "mix.g"] = (H * dv, W)
        s[p + "mix.o"] = (W, H * dv)
        if ml:
            for e in range(ml["router"]["experts"]):
                s["%smlp.e%d.gate" % (p, e)] = (ml["expert"]["ff"], W)
                s["%smlp.e%d.up" % (p, e)] = (ml["expert"]["ff"], W)
                s["%smlp.e%d.down" % (p, e)] = (W, ml["expert"]["ff"])
            s[p + "mlp.router"] = (ml["router"]["experts"], W)
            if ml.get("shared"):
                s[p + "mlp.shared.gate"] = (ml["shared"]["ff"], W)
                s[p + "mlp.shared.up"] = (ml["shared"]["ff"], W)
                s[p + "mlp.shared.down"] = (W, ml["shared"]["ff"])
                s[p + "mlp.shared.sg"] = (1, W)
    return s


def random_weights(cfg, seed, gain=1.0):
    """bf16-representable random tensors: matrices ~ N(0, gain / fan_in), norm weights small around zero (plain ones around one)."""
    g = torch.Generator().manual_seed(seed)
    w = {}
    for name, shp in tensor_shapes(cfg).items():
        if len(shp) == 1:
            t = 0.2 * torch.randn(shp, generator=g, dtype=F)
            if name.endswith(".norm") and name != "final.norm":
                t = t + 1.0
        elif name == "embed":
            t = torch.randn(shp, generator=g, dtype=F)
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


def load_model(folder):
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    with open(os.path.join(folder, "model.safetensors"), "rb") as f:
        n, = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(n))
        data = f.read()
    w = {}
    for name, m in header.items():
        if name == "__metadata__":
            continue
        a, b = m["data_offsets"]
        if m["dtype"] == "BF16":
            u = np.frombuffer(data[a:b], dtype=np.uint16).astype(np.uint32) << 16
            t = torch.from_numpy(u.view(np.float32).copy()).to(F)
        elif m["dtype"] == "F32":
            t = torch.from_numpy(np.frombuffer(data[a:b], dtype=np.float32).copy()).to(F)
        elif m["dtype"] == "I32":
            t = torch.from_numpy(np.frombuffer(data[a:b], dtype=np.int32).copy())
        else:
            raise ValueError(m["dtype"])
        w[name] = t.view(*m["shape"])
    return cfg, w


def greedy(cfg, w, prompt, n):
    """n tokens chosen by the largest logit, each from a whole forward of everything so far."""
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(torch.argmax(forward(cfg, w, toks)[-1])))
    return toks[len(prompt):]


def small_config(layers=("latent_attention", "latent_attention_2"), width=64, vocab=96, heads=2, dim=16, rot_dim=8, vdim=24, kv_rank=32,
                 q_rank=24, window=5, experts=4, top=2, ff=32, shared_ff=48, loop=None, scaling=True, limit=1.5, eps=1e-5, base=10000.0,
                 rot_dims=None, mlp_on=None):
    """A configuration whose sizes all differ from each other, so that a swapped pair shows."""
    ls = []
    for k, t in enumerate(layers):
        mx = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": 1.0 / math.sqrt(dim + rot_dim),
              "rot": {"base": base * (1 + k), "dims": rot_dims or rot_dim}}
        if t == "latent_attention":
            mx["q_rank"] = q_rank
            if scaling:
                mx["rot"]["scaling"] = {"factor": 8.0, "original": 64, "fast": 16.0, "slow": 2.0}
        else:
            mx["mask"] = {"size": window}
        ml = {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}
        if shared_ff:
            ml["shared"] = {"ff": shared_ff, "limit": limit * 0.75}
        ls.append({"type": t, "mixer": mx, "mlp": ml if (mlp_on is None or mlp_on[k]) else None})
    cfg = {"architecture": "Fabolorn", "layers": ls, "norm": {"eps": eps}, "vocab": vocab, "width": width}
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg
