"""Host side of the Nizorax family (no GPU): the folder reader and the registry know the family, and the float64 restatement's own invariants --
the things the GPU tests lean on: causality, the carried pieces of every mechanism (convolution inputs, cached keys, recurrent state), the rotation,
the choice of experts."""
import ctypes as C
import json
import math
import os
import sys

import numpy as np
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import nizorax_oracle as O  # noqa: E402
from ntransformer_amd import _lib  # noqa: E402


def describe(path):
    L = _lib.lib()
    L.nt_model_folder_describe.argtypes = [C.c_char_p, C.c_char_p, C.c_int]
    n = L.nt_model_folder_describe(path.encode(), None, 0)
    assert n >= 0
    buf = C.create_string_buffer(n + 1)
    assert L.nt_model_folder_describe(path.encode(), buf, n + 1) == n
    return json.loads(buf.value.decode())


def test_a_written_folder_is_described_and_its_family_is_built_in(tmp_path):
    cfg = O.small_config(layers=("attention", "lightning", "attention"), mlps=("moe", "dense", None), loop=(0, 2, 2))
    w = O.random_weights(cfg, 3)
    O.save_model(str(tmp_path / "m"), cfg, w)
    d = describe(str(tmp_path / "m"))
    assert d["architecture"] == "Nizorax" and d["family_built_in"] is True and {"Nizorax", "Fabolorn"} <= set(d["families"])
    got = {t["name"]: tuple(t["shape"]) for t in d["tensors"]}
    assert got == {k: tuple(v.shape) for k, v in w.items()}
    assert "l2.norm2" not in got and "l2.canon2" not in got and "l1.mlp.act" in got and "l0.mlp.shared.up" in got


def test_layer_order_and_causality():
    cfg = O.small_config(layers=("attention", "lightning", "attention"), mlps=("dense", "moe", None), loop=(1, 3, 3))
    assert O.layer_runs(cfg) == [0, 1, 2, 1, 2, 1, 2]
    assert O.layer_runs(O.small_config()) == [0, 1]
    w = O.random_weights(cfg, 2)
    toks = [int(t) for t in np.random.default_rng(0).integers(0, cfg["vocab"], 14)]
    assert torch.allclose(O.forward(cfg, w, toks)[:9], O.forward(cfg, w, toks[:9]), atol=1e-10)
    lg, st = O.forward(cfg, w, toks, return_layers=True)
    assert st.shape == (7, 14, cfg["width"]) and lg.shape == (14, cfg["vocab"])


def test_every_mechanism_carries_what_a_cut_needs():
    g = torch.Generator().manual_seed(5)
    # the added convolution: the last taps - 1 inputs
    h, cw = torch.randn(11, 6, generator=g, dtype=O.F), torch.randn(6, 4, generator=g, dtype=O.F)
    whole, _ = O.conv_added(h, cw)
    a, hist = O.conv_added(h[:2], cw)
    b, hist = O.conv_added(h[2:3], cw, hist)
    c, _ = O.conv_added(h[3:], cw, hist)
    assert torch.allclose(torch.cat([a, b, c]), whole, atol=1e-12)
    assert torch.allclose(whole[0], h[0] * (1 + cw[:, 3]))                       # the first token sees zeros before it
    cfg = O.small_config()
    w = O.random_weights(cfg, 7)
    x = torch.randn(20, cfg["width"], generator=g, dtype=O.F)
    mx = cfg["layers"][0]["mixer"]
    whole, _ = O.diff_attention(x, w, "l0.mix.", mx, 1e-5)
    a, past = O.diff_attention(x[:13], w, "l0.mix.", mx, 1e-5)
    b, _ = O.diff_attention(x[13:], w, "l0.mix.", mx, 1e-5, pos=torch.arange(13, 20), past=past)
    assert torch.allclose(torch.cat([a, b]), whole, atol=1e-10)
    lx = cfg["layers"][1]["mixer"]
    whole, S = O.lightning(x, w, "l1.mix.", lx, 1e-5)
    a, S1 = O.lightning(x[:7], w, "l1.mix.", lx, 1e-5)
    b, S2 = O.lightning(x[7:], w, "l1.mix.", lx, 1e-5, state=S1)
    assert torch.allclose(torch.cat([a, b]), whole, atol=1e-10) and torch.allclose(S2, S, atol=1e-10)


def test_rotation_window_and_lambda():
    rot = {"base": 100.0, "dims": 8, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64}}
    f = O.rotary_frequencies(rot)
    f0 = O.rotary_frequencies({"base": 100.0, "dims": 8})
    assert float(f[0]) == 1.0 and float(f[3]) == float(f0[3]) / 8.0 and all(float(f0[i]) / 8.0 <= float(f[i]) <= float(f0[i]) for i in range(4))
    x = torch.randn(5, 3, 10, dtype=O.F)
    y = O.rotate_pairs(x, torch.arange(5), rot)
    assert torch.equal(y[0], x[0]) and torch.equal(y[..., 8:], x[..., 8:])
    assert torch.allclose((y[..., :8].reshape(5, 3, 4, 2) ** 2).sum(-1), (x[..., :8].reshape(5, 3, 4, 2) ** 2).sum(-1))
    q, k = torch.randn(1, 1, 8, dtype=O.F), torch.randn(1, 1, 8, dtype=O.F)
    s = lambda pq, pk: float((O.rotate_pairs(q, torch.tensor([pq]), rot) * O.rotate_pairs(k, torch.tensor([pk]), rot)).sum())   # noqa: E731
    assert abs(s(7, 3) - s(104, 100)) < 1e-9
    v = O.visible(torch.arange(6), torch.arange(6), 3)
    assert v.sum(1).tolist() == [1, 2, 3, 3, 3, 3] and bool(v[5, 3]) and not bool(v[5, 2])
    w = {"a.lq1": torch.tensor([1.0, 2.0], dtype=O.F), "a.lk1": torch.tensor([0.5, 0.25], dtype=O.F), "a.lq2": torch.zeros(2, dtype=O.F), "a.lk2": torch.ones(2, dtype=O.F)}
    assert abs(O.lambda_of(w, "a.", 0.3) - (math.e - 1.0 + 0.3)) < 1e-12


def test_choice_of_experts_and_its_margin():
    h = torch.eye(1, 6, dtype=O.F)
    wr = torch.zeros(6, 6, dtype=O.F)
    wr[:, 0] = torch.tensor([9.0, -9.0, -9.0, 3.0, 3.0, -9.0], dtype=O.F)
    ids, wts = O.route(h, wr, {"experts": 6, "top": 2, "scale": 2.0, "groups": {"count": 2, "keep": 1}})
    assert sorted(ids[0].tolist()) == [3, 4] and torch.allclose(wts[0], 2.0 * torch.sigmoid(torch.tensor([3.0, 3.0], dtype=O.F)))
    ids, _ = O.route(h, wr, {"experts": 6, "top": 2, "scale": 1.0})
    assert sorted(ids[0].tolist()) == [0, 3]                                          # without groups the towering expert is taken (ties: the lower index)
    cfg = O.small_config()
    w = O.random_weights(cfg, 1)
    assert 0.0 <= O.closest_call(cfg, w, [1, 2, 3, 4, 5]) < 1.0
    z = torch.randn(4, 9, dtype=O.F)
    assert torch.allclose(O.polynorm(z, [0.0, 0.0, 0.0, 0.5], 1e-6), torch.full((4, 9), 0.5, dtype=O.F))
    assert torch.allclose(O.polynorm(2 * z, [1.0, 1.0, 1.0, 0.0], 0.0), O.polynorm(z, [1.0, 1.0, 1.0, 0.0], 0.0))     # every term is scale-free
