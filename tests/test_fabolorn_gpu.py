"""The Fabolorn family (layer-list models: latent attention, windowed latent attention, clipped-GLU mixture of experts, a repeated span of
layers) against tests/fabolorn_oracle.py -- a float64 restatement that shares nothing with the product.  Every test makes its own small
configuration and random bf16-representable weights, writes them as a model folder and runs them through the C API (the engine's step
function, slot cache and kernels); the operator tests call include/ntk_layers.h directly.

Error measure: rms of the difference over rms of the reference.  float32 mode is held to 2e-4 (observed ~1e-6), bfloat16 mode to 4e-2."""
import json
import math
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import fabolorn_oracle as O  # noqa: E402

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TOL = {"float32": 2e-4, "bfloat16": 4e-2}


def rel(got, ref):
    got, ref = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    return float(np.sqrt(np.mean((got - ref) ** 2)) / (np.sqrt(np.mean(ref ** 2)) + 1e-30))


def make(tmp_path, cfg, seed=1, name="m"):
    w = O.random_weights(cfg, seed)
    folder = str(tmp_path / name)
    O.save_model(folder, cfg, w)
    return folder, w


def engine_for(folder, dtype="float32", ctx=512, slots=1):
    from ntransformer_amd.engine import Engine
    e = Engine()
    e.load_folder(folder, max_context=ctx, dtype=dtype, slots=slots)
    return e


def tokens_for(cfg, n, seed=0):
    return [int(t) for t in np.random.default_rng(seed).integers(0, cfg["vocab"], n)]


MIXED = dict(layers=("latent_attention", "latent_attention_2", "latent_attention"), loop=(0, 2, 2))


# ====================================================================================================================== operators
def test_norm_with_weight_around_zero_and_plain():
    from ntransformer_amd import layers as Lr
    g = np.random.default_rng(3)
    x = g.standard_normal((5, 100)) * 3
    w1, w2 = g.standard_normal(100) * 0.2, g.standard_normal(100) * 0.2
    a, b = Lr.rmsnorm_offset(x, w1, w2, 1e-5, 1.0)
    xt = torch.tensor(x.astype(np.float32), dtype=O.F)
    assert rel(a, O.norm_around_zero(xt, torch.tensor(w1.astype(np.float32), dtype=O.F), 1e-5)) < 1e-6
    assert rel(b, O.norm_around_zero(xt, torch.tensor(w2.astype(np.float32), dtype=O.F), 1e-5)) < 1e-6
    c = Lr.rmsnorm_offset(x, w1, None, 1e-5, 0.0)
    assert rel(c, O.norm_plain(xt, torch.tensor(w1.astype(np.float32), dtype=O.F), 1e-5)) < 1e-6
    # eps sits inside the root: a row of zeros stays zero, a tiny row is damped by it
    z = Lr.rmsnorm_offset(np.full((1, 100), 1e-4), w1 * 0, None, 1e-2, 1.0)
    assert abs(float(z[0, 0]) - 1e-4 / math.sqrt(1e-8 + 1e-2)) < 1e-9


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("T", [1, 3, 8, 9, 70, 130])
@pytest.mark.parametrize("N,K", [(24, 40), (130, 64), (64, 100), (96, 256)])
def test_dense_product_every_form(dtype, T, N, K):
    """the few-row form (T <= 8), the tiled forms, ragged edges in all three sizes"""
    from ntransformer_amd import layers as Lr
    g = np.random.default_rng(T * 1000 + N + K)
    x = g.standard_normal((T, K)).astype(np.float32)
    w = O.bf16_round(torch.tensor(g.standard_normal((N, K)) / math.sqrt(K))).numpy()
    y = Lr.dense(x, w, dtype)
    assert rel(y, x.astype(np.float64) @ w.T) < (1e-5 if dtype == "float32" else 1e-2)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("T,top", [(2, 2), (1, 3), (40, 2), (90, 3)])
def test_dense_grouped_and_gathered_rows(dtype, T, top):
    """rows sorted by group take their group's matrix and read the activation row of their token; empty groups cost nothing"""
    from ntransformer_amd import layers as Lr
    g = np.random.default_rng(T + top)
    E, N, K = 5, 48, 72
    x = g.standard_normal((T, K)).astype(np.float32)
    w = O.bf16_round(torch.tensor(g.standard_normal((E, N, K)) / math.sqrt(K))).numpy()
    ids = np.stack([g.permutation(E - 1)[:top] for _ in range(T)]).astype(np.int32)   # the last group stays empty
    off, order, where = Lr.moe_group(ids, E)
    flat = ids.reshape(-1)
    assert off[0] == 0 and off[-1] == T * top and off[E - 1] == off[E]
    assert sorted(order.tolist()) == list(range(T * top)) and all(where[order[r]] == r for r in range(T * top))
    for e in range(E):
        seg = order[off[e]:off[e + 1]]
        assert all(flat[p] == e for p in seg) and list(seg) == sorted(seg)      # stable
    y = Lr.dense(x, w, dtype, offsets=off, rows=order, row_div=top)
    ref = np.stack([x[order[r] // top].astype(np.float64) @ w[flat[order[r]]].T for r in range(T * top)])
    assert rel(y, ref) < (1e-5 if dtype == "float32" else 1e-2)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("T,ff,K", [(1, 20, 40), (3, 37, 64), (8, 160, 96), (6, 1, 24)])
def test_few_row_product_with_the_clipped_glu_inside(dtype, T, ff, K):
    """decoding: gate rows, up rows and the activation in one launch == the product followed by the activation"""
    from ntransformer_amd import layers as Lr
    g = np.random.default_rng(T + ff)
    x = (g.standard_normal((T, K)) * 2).astype(np.float32)
    w = O.bf16_round(torch.tensor(g.standard_normal((2 * ff, K)))).numpy()
    gu = torch.tensor(x, dtype=O.F) @ torch.tensor(w, dtype=O.F).T
    gg, uu = gu[:, :ff].clamp(max=1.5), gu[:, ff:].clamp(-1.5, 1.5)
    ref = gg * torch.sigmoid(1.702 * gg) * (uu + 1.0)
    assert rel(Lr.dense(x, w, dtype, glu_limit=1.5), ref) < (1e-5 if dtype == "float32" else 1e-2)
    assert rel(Lr.dense(x, w, dtype, glu_limit=1.5), Lr.clipped_glu(Lr.dense(x, w, dtype), 1.5)) < 1e-6


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("offset", [0.0, 1.0])
def test_few_row_product_with_the_norm_inside(dtype, offset):
    """decoding: the RMS norm of the activation row inside the product's launch == norm, then product"""
    from ntransformer_amd import layers as Lr
    g = np.random.default_rng(int(offset) + 3)
    for T, N, K in [(1, 24, 40), (5, 70, 100), (8, 33, 264)]:
        x = (g.standard_normal((T, K)) * 4).astype(np.float32)
        w = O.bf16_round(torch.tensor(g.standard_normal((N, K)) / math.sqrt(K))).numpy()
        nw = (0.2 * g.standard_normal(K) + (1.0 - offset)).astype(np.float32)
        xt = torch.tensor(x, dtype=O.F)
        normed = O.rms_unit(xt, 1e-5) * (offset + torch.tensor(nw, dtype=O.F))
        got = Lr.dense(x, w, dtype, norm_w=nw, norm_eps=1e-5, norm_offset=offset)
        assert rel(got, normed @ torch.tensor(w, dtype=O.F).T) < (1e-5 if dtype == "float32" else 1e-2)


def test_dense_accumulates_onto_start_values():
    from ntransformer_amd import layers as Lr
    g = np.random.default_rng(9)
    for T in (2, 33):
        x, w, y0 = g.standard_normal((T, 64)).astype(np.float32), g.standard_normal((40, 64)).astype(np.float32), g.standard_normal((T, 40)).astype(np.float32)
        assert rel(Lr.dense(x, w, "float32", y0=y0), y0 + x.astype(np.float64) @ w.T) < 1e-5


@pytest.mark.parametrize("scaled", [False, True])
@pytest.mark.parametrize("dims,rot_dim", [(8, 8), (4, 8), (16, 16)])
def test_rotation_normed_latent_and_cache_rows(scaled, dims, rot_dim):
    """cache rows = [latent / rms * w | rotated key part]; queries rotated in place at the tail of every head; far positions; a rotation that covers
    only the head of the rotated part leaves the rest as it was"""
    from ntransformer_amd import layers as Lr
    rot = {"base": 5000.0, "dims": dims}
    if scaled:
        rot["scaling"] = {"factor": 8.0, "original": 64, "fast": 16.0, "slow": 2.0}
    f, mag = O.rotary_frequencies(rot)
    g = np.random.default_rng(dims + rot_dim)
    T, R, H, dn, pos0 = 6, 20, 3, 12, 3000
    kv = g.standard_normal((T, R + rot_dim)).astype(np.float32)
    q = g.standard_normal((T, H * (dn + rot_dim))).astype(np.float32)
    nw = (1 + 0.2 * g.standard_normal(R)).astype(np.float32)
    cache, qrot = Lr.latent_prepare(kv, nw, 1e-5, R, rot_dim, q, H, f.numpy(), float(mag), dims, pos0)
    pos = torch.arange(pos0, pos0 + T)
    kvt, qt = torch.tensor(kv, dtype=O.F), torch.tensor(q, dtype=O.F).view(T, H, dn + rot_dim)
    assert rel(cache[pos0:, :R], O.norm_plain(kvt[:, :R], torch.tensor(nw, dtype=O.F), 1e-5)) < 1e-6
    assert rel(cache[pos0:, R:], O.rotate_pairs(kvt[:, R:], pos, rot)) < 1e-6
    want_q = qt.clone()
    want_q[:, :, dn:] = O.rotate_pairs(qt[:, :, dn:].transpose(0, 1), pos, rot).transpose(0, 1)
    assert rel(qrot, want_q.reshape(T, -1)) < 1e-6
    if dims < rot_dim:
        assert np.array_equal(cache[pos0:, R + dims:], kv[:, R + dims:])


def _attention_case(seed, T, nkeys, H, dn, dr, dv, R):
    g = np.random.default_rng(seed)
    c = g.standard_normal((nkeys, R)).astype(np.float32)
    kr = g.standard_normal((nkeys, dr)).astype(np.float32)
    uk = (g.standard_normal((H * dn, R)) / math.sqrt(R)).astype(np.float32)
    uv = (g.standard_normal((H * dv, R)) / math.sqrt(R)).astype(np.float32)
    q = g.standard_normal((T, H, dn + dr)).astype(np.float32)
    return c, kr, uk, uv, q


@pytest.mark.parametrize("window", [0, 1, 7, 64, 65])
@pytest.mark.parametrize("T,pos0", [(1, 0), (1, 200), (5, 60), (20, 0), (37, 120)])
def test_attention_both_forms_against_plain_softmax(window, T, pos0):
    """expanded keys / values and the shared-key form give the plain softmax attention; windows of one key, of a key chunk and one more"""
    from ntransformer_amd import layers as Lr
    H, dn, dr, dv, R = 3, 12, 8, 20, 24
    nkeys = pos0 + T
    c, kr, uk, uv, q = _attention_case(window * 100 + T + pos0, T, nkeys, H, dn, dr, dv, R)
    cache = np.concatenate([c, kr], axis=1)
    scale = 0.3
    t = lambda a: torch.tensor(a, dtype=O.F)   # noqa: E731
    kn, v = (t(c) @ t(uk).T).view(nkeys, H, dn), (t(c) @ t(uv).T).view(nkeys, H, dv)
    qpos, kpos = torch.arange(pos0, nkeys), torch.arange(nkeys)
    ref = O.attend(t(q)[:, :, :dn], t(q)[:, :, dn:], kn, t(kr), v, qpos, kpos, window or None, scale).reshape(T, H * dv)
    key0 = max(0, pos0 - window + 1) if window else 0
    out = Lr.latent_attention(q.reshape(T, -1), cache, R, dr, H, pos0, window, scale, K=kn[key0:].reshape(nkeys - key0, -1).numpy(),
                              V=v[key0:].reshape(nkeys - key0, -1).numpy(), key0=key0)
    assert rel(out, ref) < 1e-5
    if T <= 8:
        qf = Lr.latent_fold_query(q.reshape(T, -1), uk, H, dn, dr)
        lat = Lr.latent_attention(qf, cache, R, dr, H, pos0, window, scale)
        assert rel(Lr.latent_unfold_value(lat, uv, H), ref) < 1e-5


@pytest.mark.parametrize("far", [0, 63, 64, 500, 1234])
def test_a_far_key_among_many_is_found(far):
    """one key among 1300 gets a score that towers over the rest: the result is that key's value (split walk and merge included)"""
    from ntransformer_amd import layers as Lr
    H, dn, dr, dv, R, n = 2, 8, 4, 8, 16, 1300
    c, kr, uk, uv, q = _attention_case(far, 1, n, H, dn, dr, dv, R)
    kr *= 0.01
    kr[far] = 0.0
    kr[far, 0] = 30.0
    q[:, :, dn] = 30.0                                  # 900 against scores of a few units
    cache = np.concatenate([c, kr], axis=1)
    qf = Lr.latent_fold_query(q.reshape(1, -1), uk, H, dn, dr)
    lat = Lr.latent_attention(qf, cache, R, dr, H, n - 1, 0, 1.0).reshape(H, R)
    for h in range(H):
        assert np.allclose(lat[h], c[far], atol=1e-4)


@pytest.mark.parametrize("T", [1, 20])
def test_window_edge_keys_in_and_out(T):
    """the key just inside the window dominates if it is seen; the key just outside would dominate even more if it leaked"""
    from ntransformer_amd import layers as Lr
    H, dn, dr, dv, R, window, pos0 = 2, 8, 4, 8, 16, 70, 150
    n = pos0 + T
    c, kr, uk, uv, q = _attention_case(T, T, n, H, dn, dr, dv, R)
    kr *= 0.01
    q[:, :, dn] = 30.0
    last = n - 1
    kr[last - window + 1, 0] = 20.0                     # inside for the last query
    kr[last - window, 0] = 40.0                         # outside for the last query (inside for the one before)
    cache = np.concatenate([c, kr], axis=1)
    t = lambda a: torch.tensor(a, dtype=O.F)   # noqa: E731
    kn, v = (t(c) @ t(uk).T).view(n, H, dn), (t(c) @ t(uv).T).view(n, H, dv)
    ref = O.attend(t(q)[:, :, :dn], t(q)[:, :, dn:], kn, t(kr), v, torch.arange(pos0, n), torch.arange(n), window, 1.0).reshape(T, H * dv)
    assert np.allclose(ref[-1].view(H, dv)[0].numpy(), v[last - window + 1, 0].numpy(), atol=1e-6)
    if T <= 8:
        qf = Lr.latent_fold_query(q.reshape(T, -1), uk, H, dn, dr)
        out = Lr.latent_unfold_value(Lr.latent_attention(qf, cache, R, dr, H, pos0, window, 1.0), uv, H)
    else:
        key0 = pos0 - window + 1
        out = Lr.latent_attention(q.reshape(T, -1), cache, R, dr, H, pos0, window, 1.0, K=kn[key0:].reshape(n - key0, -1).numpy(),
                                  V=v[key0:].reshape(n - key0, -1).numpy(), key0=key0)
    assert rel(out, ref) < 1e-5


def test_router_choice_weights_and_shared_gate():
    from ntransformer_amd import layers as Lr
    g = np.random.default_rng(5)
    T, n, E, top = 11, 72, 6, 3
    h = g.standard_normal((T, n)).astype(np.float32)
    wr, ws = g.standard_normal((E, n)).astype(np.float32) * 0.3, g.standard_normal(n).astype(np.float32) * 0.1
    ids, wts, sg = Lr.moe_route(h, wr, top, ws)
    ridx, rw = O.route(torch.tensor(h, dtype=O.F), torch.tensor(wr, dtype=O.F), top)
    assert np.array_equal(ids, ridx.numpy())
    assert rel(wts, rw) < 1e-5 and np.allclose(wts.sum(1), 1.0, atol=1e-6)
    assert rel(sg, torch.sigmoid(torch.tensor(h, dtype=O.F) @ torch.tensor(ws, dtype=O.F))) < 1e-5
    # top == experts: everything chosen, weights are the softmax itself
    ids, wts, _ = Lr.moe_route(h, wr, E)
    assert sorted(ids[0].tolist()) == list(range(E)) and np.allclose(wts.sum(1), 1.0, atol=1e-6)


def test_clipped_glu_and_weighted_sum():
    from ntransformer_amd import layers as Lr
    g = np.random.default_rng(6)
    gu = (g.standard_normal((9, 2 * 20)) * 3).astype(np.float32)     # many values beyond the limit on both sides
    a = Lr.clipped_glu(gu, 1.25)
    gg, uu = torch.tensor(gu[:, :20], dtype=O.F).clamp(max=1.25), torch.tensor(gu[:, 20:], dtype=O.F).clamp(-1.25, 1.25)
    assert rel(a, gg * torch.sigmoid(1.702 * gg) * (uu + 1.0)) < 1e-6
    T, top, n = 4, 2, 24
    x, mix, d, sh = (g.standard_normal(s).astype(np.float32) for s in ((T, n), (T, n), (T * top, n), (T, n)))
    where, wts, sgate = g.permutation(T * top).astype(np.int32), g.random((T, top)).astype(np.float32), g.random(T).astype(np.float32)
    out = Lr.moe_combine(x, mix, d, where, wts, sh, sgate)
    ref = x + mix + sum(wts[:, s:s + 1] * d[where.reshape(T, top)[:, s]] for s in range(top)) + sgate[:, None] * sh
    assert rel(out, ref) < 1e-6


# ====================================================================================================================== the model
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompt_logits_and_every_layer_run(tmp_path, dtype):
    cfg = O.small_config(**MIXED)
    folder, w = make(tmp_path, cfg)
    e = engine_for(folder, dtype)
    toks = tokens_for(cfg, 45)
    ref, layers = O.forward(cfg, w, toks, return_layers=True)
    s = e.seq_acquire()
    e.seq_capture(True)
    got = e.seq_forward(s, toks)
    cap = e.seq_captured(len(toks))
    assert cap.shape[0] == 5 == e.layer_runs                       # (0, 1) twice, then 2
    for r in range(cap.shape[0]):
        assert rel(cap[r], layers[r]) < TOL[dtype], "layer run %d" % r
    assert rel(got, ref) < TOL[dtype]


def test_first_tokens_and_single_token_sequences(tmp_path):
    cfg = O.small_config(**MIXED)
    folder, w = make(tmp_path, cfg, seed=2)
    e = engine_for(folder)
    for toks in ([7], [7, 7], [0, cfg["vocab"] - 1, 3]):
        s = e.seq_acquire()
        assert rel(e.seq_forward(s, toks), O.forward(cfg, w, toks)) < TOL["float32"]
        e.seq_release(s)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prefill_against_token_by_token_and_portions(tmp_path, dtype):
    """the same sequence whole, one token at a time, and in portions of changing size down to two tokens: same logits at every position.
    150 tokens with a window of 70: portions start and end inside the window, across the 64-key chunks and across the switch between the
    few-token form (<= 8) and the prompt form of the mixer"""
    cfg = O.small_config(window=70, **MIXED)
    folder, w = make(tmp_path, cfg, seed=3)
    e = engine_for(folder, dtype)
    toks = tokens_for(cfg, 150, seed=4)
    ref = O.forward(cfg, w, toks).numpy()
    s = e.seq_acquire()
    whole = e.seq_forward(s, toks)
    e.seq_release(s)
    assert rel(whole, ref) < TOL[dtype]
    s = e.seq_acquire()
    one = np.concatenate([e.seq_forward(s, toks[i:i + 1]) for i in range(len(toks))])
    e.seq_release(s)
    assert rel(one, ref) < TOL[dtype]
    worst = np.max(np.sqrt(np.mean((one - ref) ** 2, axis=1)) / np.sqrt(np.mean(ref ** 2)))
    assert worst < 3 * TOL[dtype]                                  # no single position stands out (a window edge, a chunk edge)
    s = e.seq_acquire()
    parts, at = [], 0
    for n in [2, 9, 3, 8, 17, 2, 30, 1, 5, 64, 2, 7]:
        parts.append(e.seq_forward(s, toks[at:at + n]))
        at += n
    assert at == len(toks) and e.seq_length(s) == at
    cut = np.concatenate(parts)
    assert rel(cut, ref) < TOL[dtype]
    assert np.max(np.sqrt(np.mean((cut - ref) ** 2, axis=1)) / np.sqrt(np.mean(ref ** 2))) < 3 * TOL[dtype]
    if dtype == "float32":
        assert rel(cut, whole) < 1e-5 and rel(one, whole) < 1e-5


def test_wanted_places_only(tmp_path):
    cfg = O.small_config(**MIXED)
    folder, w = make(tmp_path, cfg, seed=5)
    e = engine_for(folder)
    toks = tokens_for(cfg, 30, seed=6)
    ref = O.forward(cfg, w, toks).numpy()
    s = e.seq_acquire()
    a = e.seq_forward(s, toks[:20], want=[0, 7, 19])
    b = e.seq_forward(s, toks[20:], want=[])
    assert b.shape == (0, cfg["vocab"]) and e.seq_length(s) == 30
    assert rel(a, ref[[0, 7, 19]]) < TOL["float32"]


def test_slots_side_by_side_freed_and_used_again(tmp_path):
    """two sequences of unequal length interleaved in two slots equal each alone; a released slot serves the next sequence with no trace of
    the last one (its longer cache rows are still there)"""
    cfg = O.small_config(window=6, **MIXED)
    folder, w = make(tmp_path, cfg, seed=7)
    e = engine_for(folder, slots=2)
    ta, tb, tc = tokens_for(cfg, 60, 1), tokens_for(cfg, 23, 2), tokens_for(cfg, 9, 3)
    ra, rb, rc = (O.forward(cfg, w, t).numpy() for t in (ta, tb, tc))
    a, b = e.seq_acquire(), e.seq_acquire()
    assert {a, b} == {0, 1}
    with pytest.raises(Exception):
        e.seq_acquire()                                             # both taken
    ga = [e.seq_forward(a, ta[:25])]
    gb = [e.seq_forward(b, tb[:3])]
    ga.append(e.seq_forward(a, ta[25:26]))
    gb.append(e.seq_forward(b, tb[3:]))
    ga.append(e.seq_forward(a, ta[26:]))
    assert rel(np.concatenate(ga), ra) < TOL["float32"] and rel(np.concatenate(gb), rb) < TOL["float32"]
    e.seq_release(a)
    c = e.seq_acquire()
    assert c == a and e.seq_length(c) == 0
    assert rel(e.seq_forward(c, tc), rc) < TOL["float32"]
    # cutting a sequence back and running on from there
    e.seq_truncate(b, 10)
    assert rel(e.seq_forward(b, tb[10:]), rb[10:]) < TOL["float32"]


@pytest.mark.parametrize("kw", [
    dict(layers=("latent_attention_2",), heads=1, top=1, experts=1, shared_ff=0, window=1),                 # one of everything, a window of one key
    dict(layers=("latent_attention", "latent_attention"), top=4, experts=4, dim=8, vdim=8, rot_dim=8, kv_rank=8, q_rank=8, ff=8, shared_ff=8),   # equal sizes
    dict(layers=("latent_attention_2", "latent_attention", "latent_attention_2"), loop=(1, 3, 3), rot_dims=4, scaling=False, width=40, heads=3,
         dim=10, vdim=6, kv_rank=14, q_rank=18, ff=20, shared_ff=12, vocab=50),                                  # a layer ahead of the repeated span, odd sizes
    dict(layers=("latent_attention", "latent_attention_2"), mlp_on=(False, True), loop=(0, 1, 1)),           # a layer without feed-forward, one pass
    dict(layers=("latent_attention", "latent_attention_2"), width=128, heads=4, dim=32, rot_dim=16, vdim=72, kv_rank=80, q_rank=48, experts=9, top=3,
         ff=56, shared_ff=24, window=33),                                                                        # value rows and latents past one 64-column slab
    dict(layers=("latent_attention", "latent_attention_2"), width=128, heads=3, dim=128, rot_dim=64, vdim=128, kv_rank=512, q_rank=96, experts=4, top=2,
         ff=64, shared_ff=64, window=20, vocab=64),                                                              # head sizes of a full-sized model: 8 latent slabs, 2 latent columns per thread
    dict(layers=("latent_attention_2", "latent_attention"), experts=130, top=9, ff=8, shared_ff=0, window=1000, heads=5, loop=(0, 2, 3)),   # many experts (three per lane),
                                                                                                                 # more picks than few-row products take, a window wider than the sequence
])
def test_other_sizes_and_degenerate_values(tmp_path, kw):
    cfg = O.small_config(**kw)
    folder, w = make(tmp_path, cfg, seed=11)
    toks = tokens_for(cfg, 40, seed=12)
    ref = O.forward(cfg, w, toks).numpy()
    for dtype in ("float32", "bfloat16"):
        e = engine_for(folder, dtype)
        s = e.seq_acquire()
        got = np.concatenate([e.seq_forward(s, toks[:29]), e.seq_forward(s, toks[29:31])] + [e.seq_forward(s, toks[i:i + 1]) for i in range(31, 40)])
        assert rel(got, ref) < TOL[dtype], dtype
        e.close()


def test_long_decoding_from_one_token(tmp_path):
    cfg = O.small_config(window=40, **MIXED)
    folder, w = make(tmp_path, cfg, seed=13)
    e = engine_for(folder)
    toks = tokens_for(cfg, 200, seed=14)
    ref = O.forward(cfg, w, toks).numpy()
    s = e.seq_acquire()
    got = np.concatenate([e.seq_forward(s, toks[i:i + 1]) for i in range(len(toks))])
    err = np.sqrt(np.mean((got - ref) ** 2, axis=1)) / np.sqrt(np.mean(ref ** 2))
    assert err.max() < TOL["float32"], int(err.argmax())


def test_greedy_generation_through_the_engine_and_the_command_line(tmp_path):
    cfg = O.small_config(**MIXED)
    folder, w = make(tmp_path, cfg, seed=15)
    prompt = tokens_for(cfg, 12, seed=16)
    want = O.greedy(cfg, w, prompt, 10)
    e = engine_for(folder)
    assert e.is_sequence_model and e.vocab_size == cfg["vocab"] and e.hidden_size == cfg["width"] and e.n_layers == 3
    got = e.generate_tokens(prompt, 10, temperature=0.0, stop_at_eos=False)
    assert got == want
    st = e.stats()
    assert st.prompt_tokens == 12 and st.gen_tokens == 9
    assert e.generate_tokens(prompt, 10, temperature=0.0, stop_at_eos=False) == want      # the slot came back
    # sampling goes through the engine's sampler: same seed, same draws
    a = e.generate_tokens(prompt, 8, temperature=0.9, top_k=20, top_p=0.95, seed=5, stop_at_eos=False)
    assert a == e.generate_tokens(prompt, 8, temperature=0.9, top_k=20, top_p=0.95, seed=5, stop_at_eos=False) and len(a) == 8
    # the reference's forward(tokens, start_pos) keeps slot 0 for itself from its first call on
    assert rel(e.forward(prompt, 0), O.forward(cfg, w, prompt)[-1]) < TOL["float32"]
    assert rel(e.forward(prompt[8:], 8), O.forward(cfg, w, prompt)[-1]) < TOL["float32"]
    e.close()
    cli = os.path.join(ROOT, "ntransformer_amd", "ntransformer")
    r = subprocess.run([cli, "-m", folder, "--dtype", "float32", "--tokens", ",".join(map(str, prompt)), "-n", "10", "-t", "0", "--repeat-penalty", "1"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [int(t) for t in r.stdout.strip().splitlines()[-1].split(",")] == want


def test_trace_runner_replays_steps(tmp_path):
    """bin/trace_run: requests one after the other, portions and single tokens, logits of the wanted places per step, slots given back"""
    cfg = O.small_config(**MIXED)
    folder, w = make(tmp_path, cfg, seed=17)
    ta, tb = tokens_for(cfg, 20, 1), tokens_for(cfg, 6, 2)
    ra, rb = O.forward(cfg, w, ta).numpy(), O.forward(cfg, w, tb).numpy()
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": ta[:13], "want": [0, 12]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": ta[13:15], "want": []}], "end": []},
        {"step": 2, "entries": [{"id": "a", "tokens": ta[15:], "want": [4]}], "end": ["a"]},
        {"step": 3, "entries": [{"id": "b", "tokens": tb, "want": [5]}], "end": ["b"]},
        # two requests alive at once, portions alternating
        {"step": 4, "entries": [{"id": "c", "tokens": ta[:9], "want": []}], "end": []},
        {"step": 5, "entries": [{"id": "d", "tokens": tb[:2], "want": [1]}], "end": []},
        {"step": 6, "entries": [{"id": "c", "tokens": ta[9:], "want": [10]}, {"id": "d", "tokens": tb[2:], "want": [3]}], "end": ["c", "d"]},
    ]
    out = tmp_path / "out"
    out.mkdir()
    r = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32", "--out", str(out), "--max-tokens", "20"],
                       input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done %d" % k for k in range(7)]
    assert not (out / "1.f32").exists()
    V = cfg["vocab"]
    assert rel(np.fromfile(out / "0.f32", np.float32).reshape(-1, V), ra[[0, 12]]) < TOL["float32"]
    assert rel(np.fromfile(out / "2.f32", np.float32).reshape(-1, V), ra[[19]]) < TOL["float32"]
    assert rel(np.fromfile(out / "3.f32", np.float32).reshape(-1, V), rb[[5]]) < TOL["float32"]
    assert rel(np.fromfile(out / "5.f32", np.float32).reshape(-1, V), rb[[1]]) < TOL["float32"]
    assert rel(np.fromfile(out / "6.f32", np.float32).reshape(-1, V), np.stack([ra[19], rb[5]])) < TOL["float32"]


def test_a_folder_with_an_unknown_architecture_or_a_missing_tensor_is_refused(tmp_path):
    from ntransformer_amd.engine import Engine
    cfg = O.small_config(**MIXED)
    w = O.random_weights(cfg, 1)
    bad = dict(cfg, architecture="Nobody")
    O.save_model(str(tmp_path / "x"), bad, w)
    with pytest.raises(Exception, match="architecture"):
        Engine().load_folder(str(tmp_path / "x"))
    w2 = dict(w)
    del w2["l1.mix.dkv.norm"]
    O.save_model(str(tmp_path / "y"), cfg, w2)
    with pytest.raises(Exception, match="l1.mix.dkv.norm"):
        Engine().load_folder(str(tmp_path / "y"))
