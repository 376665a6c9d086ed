"""Host side of the model-folder path (no GPU): the config / safetensors reader behind nt_model_folder_describe, the family registry, and the
float64 restatement's own invariants (the things the GPU tests lean on)."""
import ctypes as C
import json
import os
import struct
import sys

import numpy as np
import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import fabolorn_oracle as O  # noqa: E402
from ntransformer_amd import _lib  # noqa: E402


def describe(path):
    L = _lib.lib()
    L.nt_model_folder_describe.argtypes = [C.c_char_p, C.c_char_p, C.c_int]
    n = L.nt_model_folder_describe(path.encode(), None, 0)
    if n < 0:
        return n
    buf = C.create_string_buffer(n + 1)
    assert L.nt_model_folder_describe(path.encode(), buf, n + 1) == n
    return json.loads(buf.value.decode())


def test_a_written_folder_is_described_tensor_by_tensor(tmp_path):
    cfg = O.small_config(layers=("latent_attention", "latent_attention_2"), loop=(0, 2, 2))
    w = O.random_weights(cfg, 3)
    O.save_model(str(tmp_path / "m"), cfg, w)
    d = describe(str(tmp_path / "m"))
    assert d["architecture"] == "Fabolorn" and d["family_built_in"] is True and "Fabolorn" in d["families"]
    got = {t["name"]: (tuple(t["shape"]), t["dtype"], t["nbytes"]) for t in d["tensors"]}
    assert set(got) == set(w)
    for name, t in w.items():
        assert got[name] == (tuple(t.shape), "BF16", 2 * t.numel())
    assert d["tensor_bytes"] == sum(2 * t.numel() for t in w.values())
    # what the oracle reads back is what it wrote (bf16-representable values survive exactly)
    cfg2, w2 = O.load_model(str(tmp_path / "m"))
    assert cfg2 == cfg and all(torch.equal(w2[k], w[k]) for k in w)


def test_an_unknown_architecture_is_named_but_not_built_in(tmp_path):
    cfg = dict(O.small_config(), architecture="SomethingElse")
    O.save_model(str(tmp_path / "m"), cfg, O.random_weights(cfg, 1))
    d = describe(str(tmp_path / "m"))
    assert d["architecture"] == "SomethingElse" and d["family_built_in"] is False


def _write(folder, header_bytes, data, config='{"architecture": "Fabolorn"}'):
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        f.write(config)
    with open(os.path.join(folder, "model.safetensors"), "wb") as f:
        f.write(struct.pack("<Q", len(header_bytes)) + header_bytes + data)


def test_malformed_folders_are_refused_not_read_past_their_end(tmp_path):
    ok = json.dumps({"a": {"dtype": "BF16", "shape": [2, 3], "data_offsets": [0, 12]}}).encode()
    _write(str(tmp_path / "ok"), ok, b"\0" * 12)
    assert describe(str(tmp_path / "ok"))["tensors"][0]["shape"] == [2, 3]
    assert describe(str(tmp_path / "nothing")) == -8                                   # no config.json: I/O
    _write(str(tmp_path / "short"), ok, b"\0" * 11)                                    # data ends inside the tensor
    assert describe(str(tmp_path / "short")) == -9
    bad_shape = json.dumps({"a": {"dtype": "BF16", "shape": [2, 4], "data_offsets": [0, 12]}}).encode()
    _write(str(tmp_path / "shape"), bad_shape, b"\0" * 12)                             # offsets do not fit the shape
    assert describe(str(tmp_path / "shape")) == -9
    _write(str(tmp_path / "json"), b'{"a": {"dtype": "BF16", "shape": [2, 3], ', b"\0" * 12)
    assert describe(str(tmp_path / "json")) == -9
    os.makedirs(str(tmp_path / "long"))
    with open(str(tmp_path / "long" / "config.json"), "w") as f:
        f.write("{}")
    with open(str(tmp_path / "long" / "model.safetensors"), "wb") as f:
        f.write(struct.pack("<Q", 1 << 40) + ok)                                       # header length beyond the file
    assert describe(str(tmp_path / "long")) == -9
    _write(str(tmp_path / "cfg"), ok, b"\0" * 12, config="[1, 2")                      # config is not JSON
    assert describe(str(tmp_path / "cfg")) == -9
    _write(str(tmp_path / "dtype"), json.dumps({"a": {"dtype": "Q9", "shape": [2, 3], "data_offsets": [0, 12]}}).encode(), b"\0" * 12)
    assert describe(str(tmp_path / "dtype")) == -9


def test_oracle_layer_order_and_rotation_invariants():
    cfg = O.small_config(layers=("latent_attention_2", "latent_attention", "latent_attention_2"), loop=(1, 3, 3))
    assert O.layer_runs(cfg) == [(0, False), (1, True), (2, False), (1, True), (2, False), (1, True), (2, False)]
    assert O.layer_runs(O.small_config()) == [(0, False), (1, False)]
    # a rotation keeps the length of every pair times the magnitude factor, and is the identity at position 0 (up to that factor)
    rot = {"base": 100.0, "dims": 8, "scaling": {"factor": 8.0, "original": 64, "fast": 16.0, "slow": 2.0}}
    f, mag = O.rotary_frequencies(rot)
    x = torch.randn(5, 8, dtype=O.F)
    y = O.rotate_pairs(x, torch.arange(5), rot)
    assert torch.allclose(y[0], x[0] * mag)
    assert torch.allclose((y.view(5, 4, 2) ** 2).sum(-1), (x.view(5, 4, 2) ** 2).sum(-1) * mag * mag)
    assert f[0] == 1.0 and all(f[i + 1] < f[i] for i in range(3))
    # the scores of rotated queries and keys depend on the distance of their positions only
    q, k = torch.randn(1, 8, dtype=O.F), torch.randn(1, 8, dtype=O.F)
    s = lambda pq, pk: float((O.rotate_pairs(q, torch.tensor([pq]), rot) * O.rotate_pairs(k, torch.tensor([pk]), rot)).sum())   # noqa: E731
    assert abs(s(7, 3) - s(104, 100)) < 1e-9


def test_oracle_window_and_routing_invariants():
    v = O.visible(torch.arange(6), torch.arange(6), 3)
    assert v.sum(1).tolist() == [1, 2, 3, 3, 3, 3] and bool(v[5, 3]) and not bool(v[5, 2])
    assert O.visible(torch.arange(4), torch.arange(4), None).sum().item() == 10
    h, wr = torch.randn(7, 12, dtype=O.F), torch.randn(5, 12, dtype=O.F)
    idx, wt = O.route(h, wr, 2)
    full = torch.softmax(h @ wr.T, -1)
    assert torch.allclose(wt.sum(-1), torch.ones(7, dtype=O.F))
    assert all(set(idx[t].tolist()) == set(torch.argsort(full[t], descending=True)[:2].tolist()) for t in range(7))
    # a prefix of a sequence has the logits of the whole sequence at its positions (causality of every mechanism)
    cfg = O.small_config(layers=("latent_attention", "latent_attention_2"), loop=(0, 2, 2), window=4)
    w = O.random_weights(cfg, 2)
    toks = [int(t) for t in np.random.default_rng(0).integers(0, cfg["vocab"], 14)]
    assert torch.allclose(O.forward(cfg, w, toks)[:9], O.forward(cfg, w, toks[:9]), atol=1e-10)
