"""The Nizorax family (layer-list models in the sequential form: layer norms around every sublayer, an added causal convolution on every sublayer's
input, differential window attention, lightning attention, a polynomial dense feed-forward and a grouped mixture of gated experts, a repeated span of
layers) against tests/nizorax_oracle.py -- a float64 restatement that shares nothing with the product.  Every test makes its own small configuration
and random bf16-representable weights, writes them as a model folder and runs them through the C API (the engine's step function, slot cache and state
and kernels); the operator tests call include/ntk_layers.h directly.

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
import nizorax_oracle as O  # noqa: E402

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TOL = {"float32": 2e-4, "bfloat16": 4e-2}


def rel(got, ref):
    got, ref = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    return float(np.sqrt(np.mean((got - ref) ** 2)) / (np.sqrt(np.mean(ref ** 2)) + 1e-30))


def row_err(got, ref):
    got, ref = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    return np.sqrt(np.mean((got - ref) ** 2, axis=1)) / np.sqrt(np.mean(ref ** 2))


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


def t64(a):
    return torch.tensor(np.asarray(a, np.float32), dtype=O.F)


MIXED = dict(layers=("lightning", "attention", "lightning", "attention"), mlps=("moe", "dense", "moe", "dense"), loop=(1, 3, 2))


# ====================================================================================================================== operators
def test_layer_norm_with_bias_and_onto_the_stream():
    from ntransformer_amd import layers as Lr
    g = np.random.default_rng(3)
    x = (g.standard_normal((5, 100)) * 3 + 2).astype(np.float32)
    w, b = (1 + 0.2 * g.standard_normal(100)).astype(np.float32), (0.3 * g.standard_normal(100)).astype(np.float32)
    ref = O.layer_norm(t64(x), t64(w), t64(b), 1e-5)
    assert rel(Lr.layernorm(x, w, b, 1e-5), ref) < 1e-6
    base = g.standard_normal((5, 100)).astype(np.float32)
    assert rel(Lr.layernorm(x, w, b, 1e-5, onto=base), t64(base) + ref) < 1e-6
    # eps sits inside the root; a constant row has no deviations and gives the bias
    z = Lr.layernorm(np.full((1, 100), 7.0, np.float32), w, b, 1e-2)
    assert np.abs(z[0] - b).max() < 1e-6
    # a large common offset must not eat the deviations (mean first, then deviations)
    y = (1000.0 + g.standard_normal((2, 300))).astype(np.float32)
    w1, b0 = np.ones(300, np.float32), np.zeros(300, np.float32)
    assert rel(Lr.layernorm(y, w1, b0, 1e-6), O.layer_norm(t64(y), t64(w1), t64(b0), 1e-6)) < 1e-4


@pytest.mark.parametrize("taps", [1, 2, 3, 5])
def test_added_convolution_carries_its_last_inputs_across_portions(taps):
    """whole == portions of every size (also shorter than the carried inputs); a sequence's start reads zeros, whatever the state held"""
    from ntransformer_amd import layers as Lr
    g = np.random.default_rng(taps)
    T, n = 23, 70
    x = (g.standard_normal((T, n)) * 2).astype(np.float32)
    w, b = (1 + 0.2 * g.standard_normal(n)).astype(np.float32), (0.3 * g.standard_normal(n)).astype(np.float32)
    cw = O.bf16_round(torch.tensor(0.5 * g.standard_normal((n, taps)))).numpy().astype(np.float32)
    ref, last = O.conv_added(O.layer_norm(t64(x), t64(w), t64(b), 1e-5), t64(cw))
    garbage = np.full((max(taps - 1, 1), n), 1e6, np.float32)       # what a freed slot may hold
    whole, st = Lr.norm_conv(x, w, b, 1e-5, cw, garbage.copy(), 0)
    assert rel(whole, ref) < 1e-6
    if taps > 1:
        assert rel(st, last) < 1e-6
    parts, at, st = [], 0, garbage.copy()
    for k in [1, 1, 2, 1, 7, 3, 8]:
        o, st = Lr.norm_conv(x[at:at + k], w, b, 1e-5, cw, st if taps > 1 else garbage.copy(), at)
        parts.append(o)
        at += k
    assert at == T and rel(np.concatenate(parts), ref) < 1e-6
    # the tap of the present token is the last column: with only it set, out = h * (1 + w)
    only = np.zeros((n, taps), np.float32)
    only[:, taps - 1] = 0.25
    o, _ = Lr.norm_conv(x, w, b, 1e-5, only, garbage.copy(), 0)
    assert rel(o, 1.25 * O.layer_norm(t64(x), t64(w), t64(b), 1e-5)) < 1e-6


@pytest.mark.parametrize("taps", [1, 2, 4])
@pytest.mark.parametrize("n", [70, 1000, 4500])
def test_the_seam_between_sublayers_in_one_call(taps, n):
    """the owed sublayer output onto the stream, the next norm, the convolution and its carried inputs: token by token (one launch each), in portions
    (two launches), and against the pieces one after the other; rows wider than a thread keeps in registers"""
    from ntransformer_amd import layers as Lr
    g = np.random.default_rng(taps + n)
    T = 9
    x = (g.standard_normal((T, n)) * 2).astype(np.float32)
    y = (g.standard_normal((T, n)) * 3 + 1).astype(np.float32)
    w, b, ow, ob = ((k + 0.2 * g.standard_normal(n)).astype(np.float32) for k in (1, 0, 1, 0))
    cw = O.bf16_round(torch.tensor(0.5 * g.standard_normal((n, taps)))).numpy().astype(np.float32)
    xs = t64(x) + O.layer_norm(t64(y), t64(ow), t64(ob), 1e-5)
    ref, last = O.conv_added(O.layer_norm(xs, t64(w), t64(b), 1e-5), t64(cw))
    garbage = np.full((max(taps - 1, 1), n), 1e6, np.float32)
    for cuts in ([T], [1] * T, [1, 3, 1, 4]):
        outs, news, at, st = [], [], 0, garbage.copy()
        for k in cuts:
            o, xn, st2 = Lr.sandwich_norm_conv(x[at:at + k], w, b, 1e-5, cw, st, at, owed=y[at:at + k], owed_w=ow, owed_b=ob)
            if taps > 1:
                st = st2
            outs.append(o)
            news.append(xn)
            at += k
        assert rel(np.concatenate(outs), ref) < 1e-6, cuts
        assert rel(np.concatenate(news), xs) < 1e-6
        if taps > 1:
            assert rel(st, last) < 1e-6
    plain, xn, _ = Lr.sandwich_norm_conv(x, w, b, 1e-5, cw, garbage.copy(), 0)          # nothing owed: the stream stays as it is
    assert np.array_equal(xn, x) and rel(plain, O.conv_added(O.layer_norm(t64(x), t64(w), t64(b), 1e-5), t64(cw))[0]) < 1e-6


def test_polynomial_activation_and_gated_norm():
    from ntransformer_amd import layers as Lr
    g = np.random.default_rng(5)
    for T, n in [(1, 40), (6, 300), (3, 1031)]:
        z = (g.standard_normal((T, n)) * 1.5).astype(np.float32)
        coef = [0.8, -0.4, 0.25, 0.1]
        assert rel(Lr.polynorm(z, coef, 1e-5), O.polynorm(t64(z), coef, 1e-5)) < 1e-6
        # each term alone: the powers are normed separately, the constant is added once
        for k in range(3):
            c = [0.0, 0.0, 0.0, 0.0]
            c[k] = 1.0
            assert rel(Lr.polynorm(z, c, 1e-5), O.unit_rms(t64(z) ** (k + 1), 1e-5)) < 1e-6
        assert np.abs(Lr.polynorm(z, [0, 0, 0, 0.7], 1e-5) - 0.7).max() < 1e-7
        w, gt = (1 + 0.2 * g.standard_normal(n)).astype(np.float32), g.standard_normal((T, n)).astype(np.float32)
        assert rel(Lr.gated_rmsnorm(z, w, gt, 1e-5), O.unit_rms(t64(z), 1e-5) * t64(w) * torch.sigmoid(t64(gt))) < 1e-6
        assert rel(Lr.gated_rmsnorm(z, w, None, 1e-5), O.unit_rms(t64(z), 1e-5) * t64(w)) < 1e-6


@pytest.mark.parametrize("scaled", [False, True])
@pytest.mark.parametrize("dims,dn", [(8, 8), (4, 10), (16, 16), (0, 6)])
def test_rotation_of_every_map_and_cache_rows(scaled, dims, dn):
    from ntransformer_amd import layers as Lr
    g = np.random.default_rng(dims + dn)
    H, G, maps, dv, T, pos0 = 4, 2, 2, 7, 5, 37
    rot = {"base": 10000.0, "dims": dims}
    if scaled:
        rot["scaling"] = {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 32}
    q, k, v = (g.standard_normal((T, n)).astype(np.float32) for n in (H * maps * dn, G * maps * dn, G * dv))
    freq = O.rotary_frequencies(rot).numpy() if dims else np.zeros(0)
    cache, qr = Lr.window_prepare(q, k, v, H, G, maps, dn, dv, freq, dims, pos0)
    pos = torch.arange(pos0, pos0 + T)
    assert rel(qr, O.rotate_pairs(t64(q).view(T, H * maps, dn), pos, rot).reshape(T, -1)) < 1e-6
    assert rel(cache[pos0:, :G * maps * dn], O.rotate_pairs(t64(k).view(T, G * maps, dn), pos, rot).reshape(T, -1)) < 1e-6
    assert np.array_equal(cache[pos0:, G * maps * dn:], v) and not cache[:pos0].any()
    if scaled and dims >= 8:
        f0, f1 = O.rotary_frequencies({"base": 10000.0, "dims": dims}), O.rotary_frequencies(rot)
        assert float(f1[0]) == float(f0[0]) and abs(float(f1[-1]) - float(f0[-1]) / 4.0) < 1e-12     # short waves stay, long ones are slowed


def _plain_attention(q, kc, vc, H, G, maps, dn, dv, pos0, window, scale, lam, sub_norm, eps, out_scale):
    T, P = q.shape[0], kc.shape[0]
    q, kc, vc = t64(q).view(T, H, maps, dn), t64(kc).view(P, G, maps, dn), t64(vc).view(P, G, dv)
    ok = O.visible(torch.arange(pos0, pos0 + T), torch.arange(P), window)
    out = torch.zeros(T, H, dv, dtype=O.F)
    for h in range(H):
        gq = h // (H // G)
        a = []
        for m in range(maps):
            s = (q[:, h, m] @ kc[:, gq, m].T * scale).masked_fill(~ok, -math.inf)
            a.append(torch.softmax(s, -1) @ vc[:, gq])
        o = a[0] - lam * a[1] if maps == 2 else a[0]
        if sub_norm:
            o = O.unit_rms(o, eps)
        out[:, h] = o * out_scale
    return out.reshape(T, H * dv)


@pytest.mark.parametrize("window", [0, 1, 7, 64, 65])
@pytest.mark.parametrize("T,pos0", [(1, 0), (1, 200), (5, 60), (20, 0), (37, 120)])
@pytest.mark.parametrize("H,G,maps", [(4, 2, 2), (3, 3, 1), (6, 1, 2)])
def test_window_attention_against_plain_softmax(window, T, pos0, H, G, maps):
    from ntransformer_amd import layers as Lr
    g = np.random.default_rng(window * 100 + T + pos0 + H)
    dn, dv, P = 12, 20, pos0 + T
    q = g.standard_normal((T, H * maps * dn)).astype(np.float32)
    kc, vc = g.standard_normal((P, G * maps * dn)).astype(np.float32), g.standard_normal((P, G * dv)).astype(np.float32)
    cache = np.concatenate([kc, vc], 1)
    ref = _plain_attention(q, kc, vc, H, G, maps, dn, dv, pos0, window, 0.4, 0.7, maps == 2, 1e-5, 0.45)
    for split in (False, True):
        got = Lr.window_attention(q, cache, H, G, maps, dn, dv, pos0, window, 0.4, lam=0.7, sub_norm=maps == 2, eps=1e-5, out_scale=0.45, split=split)
        assert rel(got, ref) < 2e-5, split


@pytest.mark.parametrize("dn,dv", [(128, 128), (70, 130), (5, 3)])
def test_window_attention_head_sizes_past_one_slab(dn, dv):
    from ntransformer_amd import layers as Lr
    g = np.random.default_rng(dn)
    H, G, maps, T, pos0 = 4, 2, 2, 9, 100
    P = pos0 + T
    q = (g.standard_normal((T, H * maps * dn)) / math.sqrt(dn)).astype(np.float32)
    kc, vc = g.standard_normal((P, G * maps * dn)).astype(np.float32), g.standard_normal((P, G * dv)).astype(np.float32)
    ref = _plain_attention(q, kc, vc, H, G, maps, dn, dv, pos0, 50, 1.0, 0.3, True, 1e-6, 1.0)
    assert rel(Lr.window_attention(q, np.concatenate([kc, vc], 1), H, G, maps, dn, dv, pos0, 50, 1.0, lam=0.3, sub_norm=True, eps=1e-6), ref) < 2e-5


@pytest.mark.parametrize("far", [0, 63, 64, 500, 1234])
@pytest.mark.parametrize("T", [1, 3])
def test_a_far_key_among_many_is_found(far, T):
    """one key whose score towers over 1300 others carries its value to the output of the first map: the walk over the chunks and the merge of the parts"""
    from ntransformer_amd import layers as Lr
    g = np.random.default_rng(far)
    H, G, maps, dn, dv, P = 2, 1, 2, 16, 8, 1300
    pos0 = P - T
    q = g.standard_normal((T, H * maps * dn)).astype(np.float32)
    kc, vc = g.standard_normal((P, G * maps * dn)).astype(np.float32) * 0.1, g.standard_normal((P, G * dv)).astype(np.float32)
    kc[far, :dn] = 6.0 * q[0, :dn]                    # map 0 of head 0 of the first query
    cache = np.concatenate([kc, vc], 1)
    got = Lr.window_attention(q, cache, H, G, maps, dn, dv, pos0, 0, 1.0, lam=0.0)
    assert np.abs(got[0, :dv] - vc[far]).max() < 1e-3
    ref = _plain_attention(q, kc, vc, H, G, maps, dn, dv, pos0, 0, 1.0, 0.0, False, 0.0, 1.0)
    assert rel(got, ref) < 2e-5


@pytest.mark.parametrize("T", [1, 20])
def test_window_edge_keys_in_and_out(T):
    """a towering key just inside the window decides the output, the same key one place further back is not seen at all"""
    from ntransformer_amd import layers as Lr
    g = np.random.default_rng(T)
    H, G, maps, dn, dv, window, P = 2, 2, 1, 8, 6, 70, 200
    pos0 = P - T
    q = g.standard_normal((T, H * dn)).astype(np.float32)
    vc = g.standard_normal((P, G * dv)).astype(np.float32)
    last = P - 1
    for back, seen in [(window - 1, True), (window, False)]:
        kc = g.standard_normal((P, G * dn)).astype(np.float32) * 0.1
        kc[last - back, :dn] = 8.0 * q[T - 1, :dn]
        got = Lr.window_attention(q, np.concatenate([kc, vc], 1), H, G, maps, dn, dv, pos0, window, 1.0)
        hit = np.abs(got[T - 1, :dv] - vc[last - back, :dv]).max() < 1e-3
        assert hit == seen
        assert rel(got, _plain_attention(q, kc, vc, H, G, maps, dn, dv, pos0, window, 1.0, 0.0, False, 0.0, 1.0)) < 2e-5


def _plain_lightning(q, k, v, decay, H, dn, dv, state=None):
    T = q.shape[0]
    q, k, v = (O.silu(t64(a)).view(T, H, -1) for a in (q, k, v))
    S = torch.zeros(H, dn, dv, dtype=O.F) if state is None else t64(state).clone()
    o = torch.zeros(T, H, dv, dtype=O.F)
    for t in range(T):
        for h in range(H):
            S[h] = decay[h] * S[h] + torch.outer(k[t, h], v[t, h])
            o[t, h] = S[h].T @ q[t, h]
    return o.reshape(T, H * dv), S


@pytest.mark.parametrize("dn,dv", [(16, 64), (10, 14), (64, 32), (130, 70), (128, 128)])
def test_lightning_recurrence_whole_portions_and_single_tokens(dn, dv):
    """the chunked walk == the recurrence token by token: whole (several chunks), in portions that cut chunks anywhere, one token at a time; a decay of 0
    forgets everything, a decay of 1 nothing; the state handed on equals the recurrence's"""
    from ntransformer_amd import layers as Lr
    g = np.random.default_rng(dn + dv)
    H, T = 4, 150
    decay = [0.0, 0.6, 0.97, 1.0]
    q, k, v = ((g.standard_normal((T, H * n)) * 0.7).astype(np.float32) for n in (dn, dn, dv))
    ref, Sref = _plain_lightning(q, k, v, decay, H, dn, dv)
    whole, S = Lr.lightning_attention(q, k, v, decay, H, dn, dv, 0)
    assert rel(whole, ref) < 1e-5 and rel(S, Sref) < 1e-5
    turn, S = Lr.lightning_attention(q, k, v, decay, H, dn, dv, 0, side_by_side=False)       # the chunks in turn by one workgroup == side by side
    assert rel(turn, ref) < 1e-5 and rel(S, Sref) < 1e-5 and rel(turn, whole) < 1e-5
    parts, at, S = [], 0, None
    for n in [2, 63, 1, 8, 57, 3, 16]:
        o, S = Lr.lightning_attention(q[at:at + n], k[at:at + n], v[at:at + n], decay, H, dn, dv, at, state=S)
        parts.append(o)
        at += n
    assert at == T and rel(np.concatenate(parts), ref) < 1e-5 and rel(S, Sref) < 1e-5
    S, one = None, []
    for t in range(40):
        o, S = Lr.lightning_attention(q[t:t + 1], k[t:t + 1], v[t:t + 1], decay, H, dn, dv, t, state=S)
        one.append(o)
    assert rel(np.concatenate(one), ref[:40]) < 1e-5
    # head 0 forgets: its output is (q . k) v of the present token alone
    qs, ks, vs = (O.silu(t64(a)) for a in (q, k, v))
    assert rel(whole[:, :dv], (qs[:, :dn] * ks[:, :dn]).sum(-1, keepdim=True) * vs[:, :dv]) < 1e-5


def test_lightning_remembers_a_far_token_and_starts_from_zeros():
    """with a decay of 1 a key written 700 tokens ago still answers a query that matches it; a sequence that starts at position 0 ignores what the state holds"""
    from ntransformer_amd import layers as Lr
    H, dn, dv, T = 1, 16, 8, 700
    g = np.random.default_rng(9)
    k = np.zeros((T, dn), np.float32)
    v = g.standard_normal((T, dv)).astype(np.float32)
    q = np.zeros((T, dn), np.float32)
    k[:, 1] = 0.05
    k[3, 0] = 3.0
    q[T - 1, 0] = 2.0
    out, S = Lr.lightning_attention(q, k, v, [1.0], H, dn, dv, 0, silu=False)
    assert np.abs(out[T - 1] - 6.0 * v[3]).max() < 1e-4
    assert np.abs(Lr.lightning_attention(q, k, v, [1.0], H, dn, dv, 0, silu=False, side_by_side=False)[0][T - 1] - 6.0 * v[3]).max() < 1e-4
    half, S1 = Lr.lightning_attention(q[:400], k[:400], v[:400], [1.0], H, dn, dv, 0, silu=False)
    rest, _ = Lr.lightning_attention(q[400:], k[400:], v[400:], [1.0], H, dn, dv, 400, state=S1, silu=False)
    assert np.abs(rest[-1] - 6.0 * v[3]).max() < 1e-4
    again, _ = Lr.lightning_attention(q, k, v, [1.0], H, dn, dv, 0, state=np.full((H, dn, dv), 1e9, np.float32), silu=False)
    assert np.array_equal(again, out)


def test_router_scores_groups_and_weights():
    from ntransformer_amd import layers as Lr
    g = np.random.default_rng(11)
    for E, top, groups, keep, n in [(6, 2, 3, 2, 48), (20, 4, 5, 2, 96), (8, 8, 1, 1, 40), (9, 2, 9, 3, 33), (130, 5, 10, 4, 64), (4, 1, 4, 1, 24), (12, 4, 3, 3, 50)]:
        h = g.standard_normal((7, n)).astype(np.float32)
        wr = (g.standard_normal((E, n)) * 2 / math.sqrt(n)).astype(np.float32)
        rt = {"experts": E, "top": top, "scale": 1.5}
        if groups > 1:
            rt["groups"] = {"count": groups, "keep": keep}
        ids, wts = Lr.moe_route_ex(h, wr, top, score=1, groups=groups, keep=keep, group_top=2, renorm=False, scale=1.5)
        rid, rw = O.route(t64(h), t64(wr), rt)
        assert np.array_equal(ids, rid.numpy()), (E, top, groups)
        assert rel(wts, rw) < 1e-6
    # a group with one towering expert and nothing else loses to a group with two good ones: the group score is the sum of the best TWO
    s = np.array([[9.0, -9.0, -9.0, 3.0, 3.0, -9.0]], np.float32)           # logits of 6 experts in 2 groups of 3
    wr = np.zeros((6, 6), np.float32)
    wr[:, 0] = s[0]
    ids, wts = Lr.moe_route_ex(np.eye(1, 6, dtype=np.float32), wr, 2, score=1, groups=2, keep=1, group_top=2, renorm=False, scale=1.0)
    assert sorted(ids[0].tolist()) == [3, 4] and abs(float(wts[0, 0]) - 1 / (1 + math.exp(-3.0))) < 1e-6
    # the softmax form with renormalised weights is what the plain router gives
    h = g.standard_normal((5, 40)).astype(np.float32)
    wr = g.standard_normal((7, 40)).astype(np.float32)
    a = Lr.moe_route(h, wr, 3)
    b = Lr.moe_route_ex(h, wr, 3, score=0, groups=1, keep=1, renorm=True, scale=1.0)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_gated_unit_alone_inside_the_few_row_product_and_the_experts_sum(dtype):
    from ntransformer_amd import layers as Lr
    g = np.random.default_rng(13)
    T, ff, K = 5, 37, 64
    x = (g.standard_normal((T, K)) * 2).astype(np.float32)
    w = O.bf16_round(torch.tensor(g.standard_normal((2 * ff, K)))).numpy()
    gu = t64(x) @ t64(w).T
    ref = O.silu(gu[:, :ff]) * gu[:, ff:]
    fused = Lr.dense(x, w, dtype, glu_limit=float("inf"), glu_alpha=1.0, glu_up_offset=0.0)
    assert rel(fused, ref) < (1e-5 if dtype == "float32" else 1e-2)
    assert rel(fused, Lr.glu(Lr.dense(x, w, dtype))) < 1e-6
    d = g.standard_normal((T * 2, 30)).astype(np.float32)
    where = g.permutation(T * 2).astype(np.int32)
    wts, sh = g.random((T, 2)).astype(np.float32), g.standard_normal((T, 30)).astype(np.float32)
    ref = np.stack([wts[t, 0] * d[where[2 * t]] + wts[t, 1] * d[where[2 * t + 1]] + sh[t] for t in range(T)])
    assert rel(Lr.moe_sum(d, where.reshape(T, 2), wts, shared=sh), ref) < 1e-6
    assert rel(Lr.moe_sum(d, where.reshape(T, 2), wts), ref - sh) < 1e-6


# ====================================================================================================================== the model
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompt_logits_and_every_layer_run(tmp_path, dtype):
    cfg = O.small_config(**MIXED)
    folder, w = make(tmp_path, cfg, seed=2)
    e = engine_for(folder, dtype)
    toks = tokens_for(cfg, 45, seed=3)
    ref, layers = O.forward(cfg, w, toks, return_layers=True)
    assert e.layer_runs == 6
    e.seq_capture(True)
    s = e.seq_acquire()
    got = e.seq_forward(s, toks)
    cap = e.seq_captured(len(toks))
    for r in range(cap.shape[0]):
        assert rel(cap[r], layers[r]) < TOL[dtype], r
    assert rel(got, ref) < TOL[dtype]


def test_first_tokens_and_single_token_sequences(tmp_path):
    cfg = O.small_config(**MIXED)
    folder, w = make(tmp_path, cfg, seed=4)
    e = engine_for(folder)
    for toks in ([7], [7, 7], [0, cfg["vocab"] - 1, 3], tokens_for(cfg, 5, 1)):
        s = e.seq_acquire()
        assert rel(e.seq_forward(s, toks), O.forward(cfg, w, toks)) < TOL["float32"]
        e.seq_release(s)
        s = e.seq_acquire()                                          # and token by token from the first one on
        got = np.concatenate([e.seq_forward(s, toks[i:i + 1]) for i in range(len(toks))])
        assert rel(got, O.forward(cfg, w, toks)) < TOL["float32"]
        e.seq_release(s)


@pytest.mark.parametrize("dtype,mlps", [("float32", MIXED["mlps"]), ("bfloat16", MIXED["mlps"]), ("bfloat16", ("dense",))])
def test_prefill_against_token_by_token_and_portions(tmp_path, dtype, mlps):
    """the same sequence whole, one token at a time, and in portions of changing size down to two tokens: same logits at every position.
    150 tokens with a window of 70: portions start and end inside the window, across the 64-key and 64-token chunks, the carried convolution
    inputs and the switch between the few-row and the tiled products.  Position by position the bfloat16 run is held to its tolerance on the model
    without a mixture (among 150 tokens some pair of expert scores is always closer than bfloat16 rounding, and the other expert is another output)"""
    cfg = O.small_config(window=70, **dict(MIXED, mlps=mlps))
    each = dtype == "float32" or "moe" not in mlps
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
    assert not each or row_err(one, ref).max() < 3 * TOL[dtype]    # no single position stands out (a window edge, a chunk edge)
    s = e.seq_acquire()
    parts, at = [], 0
    for n in [2, 9, 3, 8, 17, 2, 30, 1, 5, 64, 2, 7]:
        parts.append(e.seq_forward(s, toks[at:at + n]))
        at += n
    assert at == len(toks) and e.seq_length(s) == at
    cut = np.concatenate(parts)
    assert rel(cut, ref) < TOL[dtype]
    assert not each or row_err(cut, ref).max() < 3 * TOL[dtype]
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
    c = e.seq_forward(s, toks[:1], want=[0])                         # (one more token behind the sequence: its own logits only)
    assert b.shape == (0, cfg["vocab"]) and e.seq_length(s) == 31 and c.shape == (1, cfg["vocab"])
    assert rel(a, ref[[0, 7, 19]]) < TOL["float32"]


def test_slots_side_by_side_freed_and_used_again(tmp_path):
    """two sequences of unequal length interleaved in two slots equal each alone; a released slot serves the next sequence with no trace of the last
    one: its cache rows, its recurrent state and its convolution inputs are all still there and must not be read"""
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
    got = np.concatenate([e.seq_forward(c, tc[:1]), e.seq_forward(c, tc[1:])])     # one token first: the carried inputs of the old sequence are two deep
    assert rel(got, rc) < TOL["float32"]
    # a recurrent state cannot be cut back to the middle; to the start it can (the next token reads nothing old)
    with pytest.raises(Exception):
        e.seq_truncate(b, 10)
    e.seq_truncate(b, 0)
    assert rel(e.seq_forward(b, tc), rc) < TOL["float32"]


@pytest.mark.parametrize("kw", [
    dict(layers=("attention",), mlps=("moe",), heads=1, kv_heads=1, top=1, experts=1, groups=None, shared_ff=0, window=1, taps=1),   # one of everything, no convolution, a window of one key
    dict(layers=("lightning", "attention"), mlps=("dense", "moe"), width=16, heads=2, kv_heads=2, dim=16, vdim=16, rot_dims=16, lheads=2, ldim=16, lvdim=16,
         ff=16, eff=16, shared_ff=16, experts=4, top=4, groups=(2, 2), taps=2, decay=0.9, scaling=False),                         # equal sizes, kept groups = all, scalar decay
    dict(layers=("attention", "lightning", "attention"), mlps=("moe", "dense", None), loop=(1, 3, 3), rot_dims=4, width=40, heads=3, kv_heads=3, dim=10,
         vdim=6, lheads=5, ldim=7, lvdim=9, decay=(0.3, 0.7, 0.9, 0.99, 1.0), ff=50, vocab=50, taps=4, experts=9, groups=(3, 1), top=3),  # a layer ahead of the span, odd sizes, a layer without feed-forward
    dict(layers=("attention", "lightning"), mlps=("moe", "dense"), width=36, vocab=37, heads=2, kv_heads=1, dim=6, vdim=5, rot_dims=2, lheads=2, ldim=9, lvdim=7,
         decay=(0.8, 0.95), ff=30, eff=10, shared_ff=6, experts=4, groups=(4, 2), top=2, window=3, taps=3),                      # sizes that are multiples of nothing, groups of one expert
    dict(layers=("lightning",), mlps=(None,), taps=5, lheads=1, decay=(0.0,)),                                                     # nothing but a forgetting mixer
    dict(layers=("attention", "lightning"), mlps=("moe", "moe"), width=128, heads=6, kv_heads=2, dim=72, vdim=80, rot_dims=32, lheads=2, ldim=136, lvdim=72,
         decay=(0.95, 0.999), experts=16, top=3, groups=(2, 1), eff=24, shared_ff=40, window=33),                                  # head sizes past one 64-entry slab, the short-chunk form of the recurrence
    dict(layers=("attention", "attention"), mlps=("moe", "dense"), experts=130, top=9, groups=(13, 5), eff=8, shared_ff=0, window=1000, heads=5, kv_heads=5,
         loop=(0, 2, 3), rot_dims=0),                                                                                              # many experts, more picks than few-row products take, a window wider than the sequence, no rotation
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
    err = row_err(got, ref)
    assert err.max() < TOL["float32"], int(err.argmax())


def test_a_long_prompt_in_several_internal_passes(tmp_path):
    """more tokens than one internal pass holds: the cache rows, the recurrent state and the convolution inputs go from pass to pass"""
    cfg = O.small_config(layers=("attention", "lightning"), mlps=("dense", None), window=200, width=32, ff=40, vocab=40)
    folder, w = make(tmp_path, cfg, seed=19)
    e = engine_for(folder, ctx=1400)
    toks = tokens_for(cfg, 1100, seed=20)
    ref = O.forward(cfg, w, toks).numpy()
    s = e.seq_acquire()
    want = [0, 1, 500, 1022, 1023, 1024, 1025, 1099]
    assert rel(e.seq_forward(s, toks, want=want), ref[want]) < TOL["float32"]


def test_greedy_generation_through_the_engine_and_the_command_line(tmp_path):
    cfg = O.small_config(**MIXED)
    folder, w = make(tmp_path, cfg, seed=15)
    prompt = tokens_for(cfg, 12, seed=16)
    want = O.greedy(cfg, w, prompt, 10)
    e = engine_for(folder)
    assert e.is_sequence_model and e.vocab_size == cfg["vocab"] and e.hidden_size == cfg["width"] and e.n_layers == 4
    got = e.generate_tokens(prompt, 10, temperature=0.0, stop_at_eos=False)
    assert got == want
    st = e.stats()
    assert st.prompt_tokens == 12 and st.gen_tokens == 9
    assert e.generate_tokens(prompt, 10, temperature=0.0, stop_at_eos=False) == want      # the slot came back, its old state is not read
    a = e.generate_tokens(prompt, 8, temperature=0.9, top_k=20, top_p=0.95, seed=5, stop_at_eos=False)
    assert a == e.generate_tokens(prompt, 8, temperature=0.9, top_k=20, top_p=0.95, seed=5, stop_at_eos=False) and len(a) == 8
    # forward(tokens, start_pos) keeps slot 0 for itself: from the start, and on from where it stands
    assert rel(e.forward(prompt, 0), O.forward(cfg, w, prompt)[-1]) < TOL["float32"]
    assert rel(e.forward(prompt[:8], 0), O.forward(cfg, w, prompt[:8])[-1]) < TOL["float32"]
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
        {"step": 4, "entries": [{"id": "c", "tokens": ta[:9], "want": []}], "end": []},
        {"step": 5, "entries": [{"id": "d", "tokens": tb[:2], "want": [1]}], "end": []},
        {"step": 6, "entries": [{"id": "c", "tokens": ta[9:], "want": [10]}, {"id": "d", "tokens": tb[2:], "want": [3]}], "end": ["c", "d"]},
    ]
    V = cfg["vocab"]
    for dtype in ("float32", "bfloat16"):
        out = tmp_path / ("out_" + dtype)
        out.mkdir()
        r = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out", str(out), "--max-tokens", "20"],
                           input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600)
        assert r.returncode == 0, r.stderr[-2000:]
        assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done %d" % k for k in range(7)]
        assert not (out / "1.f32").exists()
        assert rel(np.fromfile(out / "0.f32", np.float32).reshape(-1, V), ra[[0, 12]]) < TOL[dtype]
        assert rel(np.fromfile(out / "2.f32", np.float32).reshape(-1, V), ra[[19]]) < TOL[dtype]
        assert rel(np.fromfile(out / "3.f32", np.float32).reshape(-1, V), rb[[5]]) < TOL[dtype]
        assert rel(np.fromfile(out / "5.f32", np.float32).reshape(-1, V), rb[[1]]) < TOL[dtype]
        assert rel(np.fromfile(out / "6.f32", np.float32).reshape(-1, V), np.stack([ra[19], rb[5]])) < TOL[dtype]


def test_a_folder_with_a_missing_tensor_or_a_foreign_mixer_is_refused(tmp_path):
    from ntransformer_amd.engine import Engine
    cfg = O.small_config(**MIXED)
    w = O.random_weights(cfg, 1)
    w2 = dict(w)
    del w2["l1.norm1b.b"]
    O.save_model(str(tmp_path / "y"), cfg, w2)
    with pytest.raises(Exception, match="l1.norm1b.b"):
        Engine().load_folder(str(tmp_path / "y"))
    bad = json.loads(json.dumps(cfg))
    bad["layers"][0]["type"] = "latent_attention"
    O.save_model(str(tmp_path / "z"), bad, w)
    with pytest.raises(Exception, match="mixer type"):
        Engine().load_folder(str(tmp_path / "z"))
