"""Python view of the engine C API (include/ntransformer.h): the reference's nt_engine_* surface plus the
extensions the tests and bench.py use.  Mirrors reference src/inference/engine.h (Engine::load / generate / Stats)."""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import List, Optional, Sequence

import numpy as np

from . import _lib
from ._lib import check


class GenParams(C.Structure):
    _fields_ = [("max_tokens", C.c_int), ("temperature", C.c_float), ("top_k", C.c_int), ("top_p", C.c_float),
                ("repeat_penalty", C.c_float), ("repeat_window", C.c_int), ("seed", C.c_uint64), ("stop_at_eos", C.c_int)]


class CStats(C.Structure):
    _fields_ = [("prompt_tokens", C.c_int), ("gen_tokens", C.c_int), ("prefill_ms", C.c_float), ("decode_ms", C.c_float),
                ("decode_tok_s", C.c_float)]


class SynthSpec(C.Structure):
    _fields_ = [("hidden", C.c_int), ("inter", C.c_int), ("layers", C.c_int), ("heads", C.c_int), ("kv_heads", C.c_int),
                ("vocab", C.c_int), ("ctx", C.c_int), ("eps", C.c_float), ("theta", C.c_float), ("bos", C.c_int),
                ("eos", C.c_int), ("mix", C.c_char_p), ("seed", C.c_uint64)]


PRESETS = {
    "tiny": dict(hidden=256, inter=512, layers=2, heads=4, kv_heads=2, vocab=512, ctx=256, bos=256, eos=257),
    "small": dict(hidden=1024, inter=2048, layers=4, heads=8, kv_heads=2, vocab=2048, ctx=2048, bos=256, eos=257),
    "8b": dict(hidden=4096, inter=14336, layers=32, heads=32, kv_heads=8, vocab=128256, ctx=131072, bos=128000, eos=128009),
    "70b": dict(hidden=8192, inter=28672, layers=80, heads=64, kv_heads=8, vocab=128256, ctx=131072, bos=128000, eos=128009),
}


def synth_spec(preset: str, mix: str = "Q8_0", seed: int = 20260925, layers: Optional[int] = None) -> SynthSpec:
    p = dict(PRESETS[preset])
    if layers is not None:
        p["layers"] = layers
    return SynthSpec(p["hidden"], p["inter"], p["layers"], p["heads"], p["kv_heads"], p["vocab"], p["ctx"], 1e-5, 500000.0,
                     p["bos"], p["eos"], mix.encode(), seed)


def _bind():
    L = _lib.lib()
    if getattr(L, "_engine_bound", False):
        return L
    vp, i, f = C.c_void_p, C.c_int, C.c_float
    L.nt_engine_create.restype = vp
    L.nt_engine_destroy.argtypes = [vp]
    L.nt_engine_load.argtypes = [vp, C.c_char_p]
    L.nt_engine_load_ex.argtypes = [vp, C.c_char_p, i]
    L.nt_engine_load_synthetic.argtypes = [vp, C.POINTER(SynthSpec), i]
    L.nt_engine_set_option.argtypes = [vp, C.c_char_p, C.c_char_p]
    L.nt_engine_last_error.argtypes = [vp]
    L.nt_engine_last_error.restype = C.c_char_p
    L.nt_engine_generate.argtypes = [vp, C.c_char_p, i, f, i, f]
    L.nt_engine_generate.restype = vp
    L.nt_free.argtypes = [vp]
    for n in ("vocab_size", "n_layers", "hidden_size", "max_context"):
        getattr(L, "nt_engine_" + n).argtypes = [vp]
    L.nt_gen_params_default.argtypes = [C.POINTER(GenParams)]
    L.nt_engine_generate_tokens.argtypes = [vp, C.POINTER(i), i, C.POINTER(GenParams), C.POINTER(i), i]
    L.nt_engine_last_stats.argtypes = [vp, C.POINTER(CStats)]
    L.nt_engine_forward.argtypes = [vp, C.POINTER(i), i, i, vp]
    L.nt_engine_decode_fused.argtypes = [vp, i, i, i, vp]
    L.nt_engine_tokenize.argtypes = [vp, C.c_char_p, i, C.POINTER(i), i]
    L.nt_engine_detokenize.argtypes = [vp, C.POINTER(i), i, C.c_char_p, i]
    L.nt_engine_bytes_per_token.argtypes = [vp, i]
    L.nt_engine_bytes_per_token.restype = C.c_uint64
    L.nt_engine_weight_bytes.argtypes = [vp]
    L.nt_engine_weight_bytes.restype = C.c_uint64
    L.nt_engine_resident_weight_bytes.argtypes = [vp]
    L.nt_engine_resident_weight_bytes.restype = C.c_uint64
    L.nt_engine_decode_path.argtypes = [vp]
    L.nt_engine_decode_path.restype = C.c_char_p
    L.nt_synth_write_gguf.argtypes = [C.c_char_p, C.POINTER(SynthSpec), i]
    L.nt_synth_tensor.argtypes = [C.POINTER(SynthSpec), C.c_char_p, vp, C.c_size_t, i]
    L.nt_synth_tensor.restype = C.c_int64
    L.nt_engine_decode_greedy_steps.argtypes = [vp, i, i, i, C.POINTER(i)]
    L.nt_engine_profile_token.argtypes = [vp, i, i, i, C.POINTER(f), C.POINTER(i)]
    L.nt_engine_tp_configure.argtypes = [vp, i, i]
    L.nt_engine_tp_export.argtypes = [vp, vp, C.POINTER(vp)]
    L.nt_engine_tp_connect.argtypes = [vp, vp, C.POINTER(vp)]
    L.nt_engine_tp_error.argtypes = [vp]
    L.nt_engine_tp_error.restype = C.c_uint
    L.nt_tp_slice_columns.argtypes = [vp, vp, i, C.c_int64, C.c_int64, i, i]
    L.nt_engine_debug_run_layers.argtypes = [vp, vp, i, i, i, i, i, vp]
    L.nt_engine_debug_kv_read.argtypes = [vp, i, i, i, vp, vp]
    L.nt_engine_debug_kv_write.argtypes = [vp, i, i, i, vp, vp]
    for n in ("is_sequence_model", "layer_runs", "seq_acquire"):
        getattr(L, "nt_engine_" + n).argtypes = [vp]
    L.nt_engine_seq_release.argtypes = [vp, i]
    L.nt_engine_seq_length.argtypes = [vp, i]
    L.nt_engine_seq_truncate.argtypes = [vp, i, i]
    L.nt_engine_seq_forward.argtypes = [vp, i, C.POINTER(i), i, C.POINTER(i), i, vp]
    L.nt_engine_seq_capture.argtypes = [vp, i]
    L.nt_engine_seq_copy_capture.argtypes = [vp, vp]
    L._engine_bound = True
    return L


@dataclass
class Stats:
    prompt_tokens: int
    gen_tokens: int
    prefill_ms: float
    decode_ms: float
    decode_tok_s: float


class Engine:
    def __init__(self):
        self.L = _bind()
        self.h = self.L.nt_engine_create()
        if not self.h:
            raise MemoryError("nt_engine_create")

    def close(self):
        if self.h:
            self.L.nt_engine_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def _check(self, st, what):
        if st != 0:
            raise _lib.NtkError(st, "%s: %s" % (what, (self.L.nt_engine_last_error(self.h) or b"").decode()))

    def load(self, path: str, max_context: int = 4096):
        self._check(self.L.nt_engine_load_ex(self.h, path.encode(), max_context), "load")

    def load_synthetic(self, spec: SynthSpec, max_context: int = 4096):
        self._spec = spec
        self._check(self.L.nt_engine_load_synthetic(self.h, C.byref(spec), max_context), "load_synthetic")

    # ---- tensor parallelism (include/ntransformer.h: nt_engine_tp_*) ----
    def tp_configure(self, rank: int, world: int) -> None:
        """before load(): this engine keeps slice `rank` of `world` of every projection"""
        self._check(self.L.nt_engine_tp_configure(self.h, rank, world), "tp_configure")

    def tp_export(self):
        """after load(): (64-byte hipIpc handle, raw device pointer) of this rank's communication buffer"""
        handle = C.create_string_buffer(64)
        raw = C.c_void_p()
        self._check(self.L.nt_engine_tp_export(self.h, handle, C.byref(raw)), "tp_export")
        return handle.raw, raw.value

    def tp_connect(self, handles: Optional[Sequence[bytes]] = None, raws: Optional[Sequence[int]] = None) -> None:
        """every rank, in rank order: the peers' handles (other processes) or raw pointers (ranks sharing this process)"""
        if raws is not None:
            arr = (C.c_void_p * len(raws))(*raws)
            self._check(self.L.nt_engine_tp_connect(self.h, None, arr), "tp_connect")
        else:
            blob = C.create_string_buffer(b"".join(handles), 64 * len(handles))
            self._check(self.L.nt_engine_tp_connect(self.h, blob, None), "tp_connect")

    def tp_error(self) -> int:
        return int(self.L.nt_engine_tp_error(self.h))

    def set_option(self, key: str, value) -> None:
        text = value if isinstance(value, str) else str(int(value))
        self._check(self.L.nt_engine_set_option(self.h, key.encode(), text.encode()), "set_option " + key)

    # ---- model folders (include/ntransformer.h: nt_engine_seq_*): one slot of the cache per live sequence ----
    def load_folder(self, path: str, max_context: int = 4096, dtype: str = "bfloat16", slots: int = 1) -> None:
        """a folder with config.json + model.safetensors; the model class comes from the config's architecture"""
        self.set_option("dtype", dtype)
        self.set_option("slots", slots)
        self.load(path, max_context)

    @property
    def is_sequence_model(self) -> bool:
        return bool(self.L.nt_engine_is_sequence_model(self.h))

    @property
    def layer_runs(self) -> int:
        return self.L.nt_engine_layer_runs(self.h)

    def seq_acquire(self) -> int:
        s = self.L.nt_engine_seq_acquire(self.h)
        if s < 0:
            self._check(s, "seq_acquire")
        return s

    def seq_release(self, slot: int) -> None:
        self._check(self.L.nt_engine_seq_release(self.h, slot), "seq_release")

    def seq_length(self, slot: int) -> int:
        return self.L.nt_engine_seq_length(self.h, slot)

    def seq_truncate(self, slot: int, length: int) -> None:
        self._check(self.L.nt_engine_seq_truncate(self.h, slot, length), "seq_truncate")

    def seq_forward(self, slot: int, tokens: Sequence[int], want: Optional[Sequence[int]] = None) -> np.ndarray:
        """append `tokens` to the slot; logits [len(want), vocab] of the places `want` (default: every token of this portion)"""
        want = list(range(len(tokens))) if want is None else [int(w) for w in want]
        out = np.empty((len(want), self.vocab_size), np.float32)
        arr = (C.c_int * len(tokens))(*[int(t) for t in tokens])
        warr = (C.c_int * max(len(want), 1))(*want)
        self._check(self.L.nt_engine_seq_forward(self.h, slot, arr, len(tokens), warr, len(want), out.ctypes.data_as(C.c_void_p)), "seq_forward")
        return out

    def seq_capture(self, on: bool = True) -> None:
        self._check(self.L.nt_engine_seq_capture(self.h, int(on)), "seq_capture")

    def seq_captured(self, n_tokens: int) -> np.ndarray:
        """the residual stream after every layer run of the last seq_forward: [layer runs, n_tokens, hidden]"""
        out = np.empty((self.layer_runs, n_tokens, self.hidden_size), np.float32)
        self._check(self.L.nt_engine_seq_copy_capture(self.h, out.ctypes.data_as(C.c_void_p)), "seq_copy_capture")
        return out

    @property
    def vocab_size(self): return self.L.nt_engine_vocab_size(self.h)
    @property
    def n_layers(self): return self.L.nt_engine_n_layers(self.h)
    @property
    def hidden_size(self): return self.L.nt_engine_hidden_size(self.h)

    def forward(self, tokens: Sequence[int], start_pos: int) -> np.ndarray:
        out = np.empty(self.vocab_size, np.float32)
        arr = (C.c_int * len(tokens))(*[int(t) for t in tokens])
        self._check(self.L.nt_engine_forward(self.h, arr, len(tokens), start_pos, out.ctypes.data_as(C.c_void_p)), "forward")
        return out

    def decode_fused(self, token: int, pos: int, graph: bool = False) -> np.ndarray:
        out = np.empty(self.vocab_size, np.float32)
        self._check(self.L.nt_engine_decode_fused(self.h, int(token), pos, int(graph), out.ctypes.data_as(C.c_void_p)), "decode_fused")
        return out

    # ---- parity instrumentation (include/ntransformer.h: nt_engine_debug_*) ----
    def debug_run_layers(self, hidden_in: np.ndarray, start_pos: int, first: int, count: int = 1, mode: int = 0) -> np.ndarray:
        """layers [first, first+count) on caller-supplied hidden states [T, H]; mode 0 = 1:1 launchers, 1 = fused, 2 = fused via hipGraph"""
        x = np.ascontiguousarray(hidden_in, dtype=np.float32)
        if x.ndim == 1:
            x = x[None, :]
        out = np.empty_like(x)
        self._check(self.L.nt_engine_debug_run_layers(self.h, x.ctypes.data_as(C.c_void_p), x.shape[0], start_pos, first, count, mode,
                                                      out.ctypes.data_as(C.c_void_p)), "debug_run_layers")
        return out

    def kv_read(self, layer: int, pos0: int, n: int, row_halves: int):
        """(K, V) cache rows [pos0, pos0+n) of one layer as uint16 [n, n_kv_heads * head_dim]"""
        k = np.empty((n, row_halves), np.uint16)
        v = np.empty((n, row_halves), np.uint16)
        self._check(self.L.nt_engine_debug_kv_read(self.h, layer, pos0, n, k.ctypes.data_as(C.c_void_p), v.ctypes.data_as(C.c_void_p)), "kv_read")
        return k, v

    def kv_write(self, layer: int, pos0: int, k: np.ndarray, v: np.ndarray) -> None:
        k = np.ascontiguousarray(k, dtype=np.uint16)
        v = np.ascontiguousarray(v, dtype=np.uint16)
        self._check(self.L.nt_engine_debug_kv_write(self.h, layer, pos0, k.shape[0], k.ctypes.data_as(C.c_void_p), v.ctypes.data_as(C.c_void_p)), "kv_write")

    def generate_tokens(self, prompt: Sequence[int], max_tokens: int, temperature: float = 0.0, top_k: int = 40,
                        top_p: float = 0.9, repeat_penalty: float = 1.0, repeat_window: int = 64, seed: int = 42,
                        stop_at_eos: bool = True) -> List[int]:
        p = GenParams(max_tokens, temperature, top_k, top_p, repeat_penalty, repeat_window, seed, int(stop_at_eos))
        arr = (C.c_int * len(prompt))(*[int(t) for t in prompt])
        out = (C.c_int * max(max_tokens, 1))()
        n = self.L.nt_engine_generate_tokens(self.h, arr, len(prompt), C.byref(p), out, max_tokens)
        if n < 0:
            self._check(n, "generate_tokens")
        return list(out[:n])

    def generate(self, prompt: str, max_tokens: int, temperature: float = 0.7, top_k: int = 40, top_p: float = 0.9) -> str:
        r = self.L.nt_engine_generate(self.h, prompt.encode(), max_tokens, temperature, top_k, top_p)
        if not r:
            raise _lib.NtkError(-3, "generate")
        s = C.string_at(r).decode("utf-8", "replace")
        self.L.nt_free(r)
        return s

    def decode_greedy_steps(self, token: int, pos: int, n: int) -> List[int]:
        out = (C.c_int * max(n, 1))()
        self._check(self.L.nt_engine_decode_greedy_steps(self.h, int(token), pos, n, out), "decode_greedy_steps")
        return list(out[:n])

    def profile_token(self, token: int, pos: int, coarse: bool = True):
        """One eager fused token timed with HIP events; see nt_engine_profile_token (coarse: one event per run of
        same-class launches)."""
        ms, calls = (C.c_float * 4)(), (C.c_int * 4)()
        self._check(self.L.nt_engine_profile_token(self.h, int(token), pos, 1 if coarse else 0, ms, calls), "profile_token")
        return list(ms), list(calls)

    def stats(self) -> Stats:
        s = CStats()
        self.L.nt_engine_last_stats(self.h, C.byref(s))
        return Stats(s.prompt_tokens, s.gen_tokens, s.prefill_ms, s.decode_ms, s.decode_tok_s)

    def bytes_per_token(self, pos: int = 0) -> int:
        return int(self.L.nt_engine_bytes_per_token(self.h, pos))

    def decode_path(self) -> str:
        return (self.L.nt_engine_decode_path(self.h) or b"").decode()

    def weight_bytes(self) -> int:
        return int(self.L.nt_engine_weight_bytes(self.h))

    def resident_weight_bytes(self) -> int:
        return int(self.L.nt_engine_resident_weight_bytes(self.h))

    def load_shared(self, src: "Engine", max_context: int = 4096) -> None:
        """a second sequence over the weights `src` holds resident (nt_engine_load_shared): own caches / buffers / stream; keep `src` alive"""
        self.L.nt_engine_load_shared.argtypes = [C.c_void_p, C.c_void_p, C.c_int]
        self._check(self.L.nt_engine_load_shared(self.h, src.h, max_context), "load_shared")
        self._shared_from = src

    def repacked_bytes(self) -> int:
        self.L.nt_engine_repacked_bytes.restype = C.c_uint64
        self.L.nt_engine_repacked_bytes.argtypes = [C.c_void_p]
        return int(self.L.nt_engine_repacked_bytes(self.h))

    def tokenize(self, text: str, add_bos: bool = True) -> List[int]:
        out = (C.c_int * 4096)()
        n = self.L.nt_engine_tokenize(self.h, text.encode(), int(add_bos), out, 4096)
        return list(out[:n])


def synth_write_gguf(path: str, spec: SynthSpec, nthreads: int = 0) -> None:
    check(_bind().nt_synth_write_gguf(path.encode(), C.byref(spec), nthreads), "synth_write_gguf")


def synth_tensor(spec: SynthSpec, name: str, nthreads: int = 0) -> np.ndarray:
    L = _bind()
    n = L.nt_synth_tensor(C.byref(spec), name.encode(), None, 0, nthreads)
    if n < 0:
        raise _lib.NtkError(int(n), "synth_tensor " + name)
    buf = np.empty(n, np.uint8)
    L.nt_synth_tensor(C.byref(spec), name.encode(), buf.ctypes.data_as(C.c_void_p), n, nthreads)
    return buf
