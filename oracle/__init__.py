"""ctypes binding of the CPU oracle (test infrastructure, never the product path).

Only tests/, ``__graft_entry__.smoke()`` and ``bench.py``'s ``cpu_baseline`` leg
import this package.  The library is built by ``make -C oracle`` (or
``oracle.build()``); every wrapper takes and returns numpy arrays.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from dataclasses import dataclass

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "libxabe_oracle.so")

Q6K = 0
Q8_0 = 1
BLOCK_BYTES = {Q6K: 210, Q8_0: 34}
BLOCK_ELEMENTS = {Q6K: 256, Q8_0: 32}


def build(force: bool = False) -> str:
    """Compile the oracle with gcc; returns the library path."""
    src = os.path.join(_HERE, "xabe_oracle.c")
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = C.CDLL(_LIB_PATH)
        _declare(_lib)
    return _lib


_f32p = C.POINTER(C.c_float)
_u8p = C.POINTER(C.c_uint8)
_u32p = C.POINTER(C.c_uint32)
_i32p = C.POINTER(C.c_int32)
_i8p = C.POINTER(C.c_int8)


class _Rng(C.Structure):
    _fields_ = [("state", C.c_uint64)]


class _Comparison(C.Structure):
    _fields_ = [
        ("max_abs_error", C.c_float),
        ("max_abs_error_index", C.c_size_t),
        ("max_rel_error", C.c_float),
        ("max_rel_error_index", C.c_size_t),
        ("cosine_similarity", C.c_float),
        ("non_finite_count", C.c_size_t),
        ("len", C.c_size_t),
    ]


class _MoeWeights(C.Structure):
    _fields_ = [
        ("num_experts", C.c_size_t), ("top_k", C.c_size_t), ("hidden", C.c_size_t), ("intermediate", C.c_size_t),
        ("eps", C.c_float),
        ("post_norm", _f32p), ("router_f32", _f32p), ("router_q8", _u8p),
        ("gate_quant", C.c_int), ("up_quant", C.c_int), ("down_quant", C.c_int),
        ("gate_exps", _u8p), ("up_exps", _u8p), ("down_exps", _u8p),
        ("shared_gate_inp", _f32p),
        ("sgate_quant", C.c_int), ("sup_quant", C.c_int), ("sdown_quant", C.c_int),
        ("shared_gate", _u8p), ("shared_up", _u8p), ("shared_down", _u8p),
    ]


class _MoeOutputs(C.Structure):
    _fields_ = [
        ("normed", _f32p), ("logits", _f32p), ("topk_ids", _u32p), ("topk_weights", _f32p),
        ("routed", _f32p), ("shexp", _f32p), ("gate", _f32p), ("ffn_out", _f32p), ("l_out", _f32p),
        ("seconds_dequant", C.c_double), ("seconds_matvec", C.c_double),
    ]


def _declare(L: C.CDLL) -> None:
    sz = C.c_size_t
    L.xo_rng_new.argtypes = [C.POINTER(_Rng), C.c_uint64]
    L.xo_rng_next_u64.argtypes = [C.POINTER(_Rng)]
    L.xo_rng_next_u64.restype = C.c_uint64
    L.xo_rng_next_f32.argtypes = [C.POINTER(_Rng)]
    L.xo_rng_next_f32.restype = C.c_float
    L.xo_rng_next_f32_range.argtypes = [C.POINTER(_Rng), C.c_float, C.c_float]
    L.xo_rng_next_f32_range.restype = C.c_float
    L.xo_rng_next_u32_below.argtypes = [C.POINTER(_Rng), C.c_uint32]
    L.xo_rng_next_u32_below.restype = C.c_uint32
    L.xo_rng_vec_f32.argtypes = [C.POINTER(_Rng), sz, C.c_float, C.c_float, _f32p]
    L.xo_to_f16_bits.argtypes = [C.c_float]
    L.xo_to_f16_bits.restype = C.c_uint16
    L.xo_from_f16_bits.argtypes = [C.c_uint16]
    L.xo_from_f16_bits.restype = C.c_float
    for name in ("xo_quantize_q8_0", "xo_quantize_q6_k"):
        getattr(L, name).argtypes = [_f32p, _u8p]
    for name in ("xo_dequantize_q8_0", "xo_dequantize_q6_k"):
        getattr(L, name).argtypes = [_u8p, _f32p]
    L.xo_dequantize_row.argtypes = [C.c_int, _u8p, sz, _f32p]
    L.xo_quantize_row.argtypes = [C.c_int, _f32p, sz, _u8p]
    L.xo_rms_norm.argtypes = [_f32p, _f32p, sz, C.c_float, _f32p]
    L.xo_silu.argtypes = [C.c_float]
    L.xo_silu.restype = C.c_float
    L.xo_sigmoid.argtypes = [C.c_float]
    L.xo_sigmoid.restype = C.c_float
    L.xo_swiglu.argtypes = [_f32p, _f32p, sz, _f32p]
    L.xo_sigmoid_gate.argtypes = [_f32p, _f32p, sz, _f32p]
    L.xo_residual_add.argtypes = [_f32p, _f32p, sz, _f32p]
    L.xo_gemv.argtypes = [_f32p, sz, sz, _f32p, _f32p]
    L.xo_argmax.argtypes = [_f32p, sz]
    L.xo_argmax.restype = sz
    L.xo_route_token.argtypes = [_f32p, sz, sz, _u32p, _f32p]
    L.xo_route_batch.argtypes = [_f32p, sz, sz, sz, _u32p, _f32p]
    L.xo_moe_align_block_size.argtypes = [_u32p, sz, sz, sz, sz, _u32p, _i32p, C.POINTER(sz)]
    L.xo_expert_mlp.argtypes = [_f32p, _f32p, _f32p, _f32p, sz, sz, _f32p]
    L.xo_naive_forward.argtypes = [_f32p, sz, _u32p, _f32p, sz, _f32p, _f32p, _f32p, sz, sz, _f32p]
    L.xo_grouped_forward.argtypes = [_f32p, sz, _u32p, _i32p, sz, sz, _f32p, sz, _f32p, _f32p, _f32p, sz, sz, _f32p]
    L.xo_compare.argtypes = [_f32p, _f32p, sz, C.POINTER(_Comparison)]
    for name in ("xo_sorted_capacity", "xo_expert_block_capacity"):
        getattr(L, name).argtypes = [sz, sz, sz, sz]
        getattr(L, name).restype = sz
    L.xo_max_flat_pairs.argtypes = [sz, sz]
    L.xo_max_flat_pairs.restype = sz
    L.xo_quantize_rows_q8.argtypes = [_f32p, sz, sz, _i8p, _f32p]
    L.xo_moe_block_forward.argtypes = [C.POINTER(_MoeWeights), _f32p, sz, _f32p, _f32p, C.c_int, C.POINTER(_MoeOutputs)]
    L.xo_dense_block_forward.argtypes = [sz, sz, C.c_float, _f32p, C.c_int, C.c_int, C.c_int, _u8p, _u8p, _u8p,
                                         _f32p, sz, C.c_int, _f32p, _f32p, _f32p]
    L.xo_synth_normal_f32.argtypes = [C.c_uint64, sz, C.c_float, _f32p]
    L.xo_synth_quant.argtypes = [C.c_int, C.c_uint64, sz, C.c_float, _u8p]
    L.xo_num_threads.restype = C.c_int


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def _u8(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.uint8)


def _p(a: np.ndarray, t):
    return a.ctypes.data_as(t)


# ---------------------------------------------------------------- rng
class Xorshift64Star:
    """K/rng.rs:20-55."""

    def __init__(self, seed: int):
        self._r = _Rng()
        lib().xo_rng_new(C.byref(self._r), seed & 0xFFFFFFFFFFFFFFFF)

    def next_u64(self) -> int:
        return int(lib().xo_rng_next_u64(C.byref(self._r)))

    def next_f32(self) -> float:
        return float(lib().xo_rng_next_f32(C.byref(self._r)))

    def next_f32_range(self, low: float, high: float) -> float:
        return float(lib().xo_rng_next_f32_range(C.byref(self._r), low, high))

    def next_u32_below(self, bound: int) -> int:
        return int(lib().xo_rng_next_u32_below(C.byref(self._r), bound))

    def vec_f32(self, n: int, low: float, high: float) -> np.ndarray:
        out = np.empty(n, dtype=np.float32)
        lib().xo_rng_vec_f32(C.byref(self._r), n, low, high, _p(out, _f32p))
        return out


# ---------------------------------------------------------------- f16
def to_f16_bits(x: float) -> int:
    return int(lib().xo_to_f16_bits(np.float32(x)))


def from_f16_bits(h: int) -> float:
    return float(lib().xo_from_f16_bits(h))


# ---------------------------------------------------------------- quant
def quantize_row(quant: int, x) -> np.ndarray:
    x = _f32(x).ravel()
    be, bb = BLOCK_ELEMENTS[quant], BLOCK_BYTES[quant]
    if x.size % be:
        raise ValueError("not a whole number of blocks")
    out = np.empty(x.size // be * bb, dtype=np.uint8)
    rc = lib().xo_quantize_row(quant, _p(x, _f32p), x.size, _p(out, _u8p))
    assert rc == 0
    return out


def dequantize_row(quant: int, data) -> np.ndarray:
    data = _u8(data).ravel()
    be, bb = BLOCK_ELEMENTS[quant], BLOCK_BYTES[quant]
    out = np.empty(data.size // bb * be, dtype=np.float32)
    rc = lib().xo_dequantize_row(quant, _p(data, _u8p), data.size, _p(out, _f32p))
    if rc != 0:
        raise ValueError(f"{data.size} bytes is not a whole number of {bb} B blocks")
    return out


# ---------------------------------------------------------------- norm / gemv
def rms_norm(x, weight, eps: float) -> np.ndarray:
    x, weight = _f32(x), _f32(weight)
    assert x.shape == weight.shape and x.size > 0
    y = np.empty_like(x)
    lib().xo_rms_norm(_p(x, _f32p), _p(weight, _f32p), x.size, eps, _p(y, _f32p))
    return y


def silu(x: float) -> float:
    return float(lib().xo_silu(np.float32(x)))


def sigmoid(x: float) -> float:
    return float(lib().xo_sigmoid(np.float32(x)))


def swiglu(gate, up) -> np.ndarray:
    gate, up = _f32(gate), _f32(up)
    assert gate.shape == up.shape
    out = np.empty_like(gate)
    lib().xo_swiglu(_p(gate, _f32p), _p(up, _f32p), gate.size, _p(out, _f32p))
    return out


def sigmoid_gate(x, gate) -> np.ndarray:
    x, gate = _f32(x), _f32(gate)
    out = np.empty_like(x)
    lib().xo_sigmoid_gate(_p(x, _f32p), _p(gate, _f32p), x.size, _p(out, _f32p))
    return out


def residual_add(a, b) -> np.ndarray:
    a, b = _f32(a), _f32(b)
    out = np.empty_like(a)
    lib().xo_residual_add(_p(a, _f32p), _p(b, _f32p), a.size, _p(out, _f32p))
    return out


def gemv(weight, out_dim: int, in_dim: int, x) -> np.ndarray:
    weight, x = _f32(weight).ravel(), _f32(x).ravel()
    assert weight.size == out_dim * in_dim and x.size == in_dim
    out = np.empty(out_dim, dtype=np.float32)
    lib().xo_gemv(_p(weight, _f32p), out_dim, in_dim, _p(x, _f32p), _p(out, _f32p))
    return out


def argmax(v) -> int:
    v = _f32(v)
    return int(lib().xo_argmax(_p(v, _f32p), v.size))


# ---------------------------------------------------------------- router / dispatch / gemm
def route_token(logits, k: int):
    logits = _f32(logits).ravel()
    ids = np.empty(k, dtype=np.uint32)
    w = np.empty(k, dtype=np.float32)
    rc = lib().xo_route_token(_p(logits, _f32p), logits.size, k, _p(ids, _u32p), _p(w, _f32p))
    if rc != 0:
        raise ValueError("route_token: invalid k / logits")
    return ids, w


def route_batch(logits, k: int):
    logits = _f32(logits)
    t, e = logits.shape
    ids = np.empty((t, k), dtype=np.uint32)
    w = np.empty((t, k), dtype=np.float32)
    rc = lib().xo_route_batch(_p(logits, _f32p), t, e, k, _p(ids, _u32p), _p(w, _f32p))
    if rc != 0:
        raise ValueError("route_batch: invalid k / logits")
    return ids, w


@dataclass
class MoeDispatch:
    sorted_token_ids: np.ndarray
    expert_ids: np.ndarray
    num_tokens_post_pad: int


def moe_align_block_size(topk_ids, block_size: int, num_experts: int) -> MoeDispatch:
    topk = np.ascontiguousarray(topk_ids, dtype=np.uint32)
    if topk.ndim != 2:
        raise ValueError("topk_ids must be [tokens][top_k]")
    t, k = topk.shape
    cap = t * k + num_experts * max(block_size, 1)
    sorted_ids = np.empty(cap, dtype=np.uint32)
    experts = np.empty(cap // max(block_size, 1) + 1, dtype=np.int32)
    post = C.c_size_t(0)
    rc = lib().xo_moe_align_block_size(_p(topk, _u32p), t, k, block_size, num_experts, _p(sorted_ids, _u32p),
                                       _p(experts, _i32p), C.byref(post))
    if rc != 0:
        raise ValueError("moe_align_block_size: zero block size or expert id out of range")
    n = post.value
    return MoeDispatch(sorted_ids[:n].copy(), experts[: n // block_size].copy(), n)


def expert_mlp(gate, up, down, x, hidden: int, intermediate: int) -> np.ndarray:
    gate, up, down, x = _f32(gate).ravel(), _f32(up).ravel(), _f32(down).ravel(), _f32(x).ravel()
    out = np.empty(hidden, dtype=np.float32)
    lib().xo_expert_mlp(_p(gate, _f32p), _p(up, _f32p), _p(down, _f32p), _p(x, _f32p), hidden, intermediate,
                        _p(out, _f32p))
    return out


def naive_forward(hidden_states, expert_ids, weights, gate, up, down, hidden: int, intermediate: int) -> np.ndarray:
    hs = _f32(hidden_states)
    ids = np.ascontiguousarray(expert_ids, dtype=np.uint32)
    w = _f32(weights)
    t, k = ids.shape
    gate, up, down = _f32(gate).ravel(), _f32(up).ravel(), _f32(down).ravel()
    out = np.empty((t, hidden), dtype=np.float32)
    lib().xo_naive_forward(_p(hs, _f32p), t, _p(ids, _u32p), _p(w, _f32p), k, _p(gate, _f32p), _p(up, _f32p),
                           _p(down, _f32p), hidden, intermediate, _p(out, _f32p))
    return out


def grouped_forward(hidden_states, dispatch: MoeDispatch, block_size: int, flat_weights, top_k: int, gate, up, down,
                    hidden: int, intermediate: int) -> np.ndarray:
    hs = _f32(hidden_states)
    t = hs.shape[0]
    fw = _f32(flat_weights).ravel()
    gate, up, down = _f32(gate).ravel(), _f32(up).ravel(), _f32(down).ravel()
    out = np.empty((t, hidden), dtype=np.float32)
    s = np.ascontiguousarray(dispatch.sorted_token_ids, dtype=np.uint32)
    e = np.ascontiguousarray(dispatch.expert_ids, dtype=np.int32)
    lib().xo_grouped_forward(_p(hs, _f32p), t, _p(s, _u32p), _p(e, _i32p), e.size, block_size, _p(fw, _f32p), top_k,
                             _p(gate, _f32p), _p(up, _f32p), _p(down, _f32p), hidden, intermediate, _p(out, _f32p))
    return out


# ---------------------------------------------------------------- compare
@dataclass
class ComparisonResult:
    max_abs_error: float
    max_abs_error_index: int
    max_rel_error: float
    max_rel_error_index: int
    cosine_similarity: float
    non_finite_count: int
    len: int

    def __str__(self) -> str:
        return (f"cosine={self.cosine_similarity:.6f} max_abs={self.max_abs_error:.6e} @[{self.max_abs_error_index}] "
                f"max_rel={self.max_rel_error:.6e} @[{self.max_rel_error_index}] "
                f"non_finite={self.non_finite_count}/{self.len}")


def compare(candidate, reference) -> ComparisonResult:
    c, r = _f32(candidate).ravel(), _f32(reference).ravel()
    if c.size != r.size or c.size == 0:
        raise ValueError("compare() requires equal-length, non-empty tensors")
    res = _Comparison()
    lib().xo_compare(_p(c, _f32p), _p(r, _f32p), c.size, C.byref(res))
    return ComparisonResult(res.max_abs_error, res.max_abs_error_index, res.max_rel_error, res.max_rel_error_index,
                            res.cosine_similarity, res.non_finite_count, res.len)


# ---------------------------------------------------------------- geometry
def sorted_capacity(num_experts: int, top_k: int, block_size: int, max_tokens: int) -> int:
    return int(lib().xo_sorted_capacity(num_experts, top_k, block_size, max_tokens))


def expert_block_capacity(num_experts: int, top_k: int, block_size: int, max_tokens: int) -> int:
    return int(lib().xo_expert_block_capacity(num_experts, top_k, block_size, max_tokens))


def quantize_rows_q8(x):
    x = _f32(x)
    rows, k = x.shape
    q = np.empty((rows, k), dtype=np.int8)
    s = np.empty((rows, k // 32), dtype=np.float32)
    lib().xo_quantize_rows_q8(_p(x, _f32p), rows, k, _p(q, _i8p), _p(s, _f32p))
    return q, s


# ---------------------------------------------------------------- synthetic inputs
def synth_normal_f32(seed: int, n: int, sigma: float) -> np.ndarray:
    out = np.empty(n, dtype=np.float32)
    lib().xo_synth_normal_f32(seed & 0xFFFFFFFFFFFFFFFF, n, sigma, _p(out, _f32p))
    return out


def synth_quant(quant: int, seed: int, n_elements: int, sigma: float) -> np.ndarray:
    out = np.empty(n_elements // BLOCK_ELEMENTS[quant] * BLOCK_BYTES[quant], dtype=np.uint8)
    rc = lib().xo_synth_quant(quant, seed & 0xFFFFFFFFFFFFFFFF, n_elements, sigma, _p(out, _u8p))
    if rc != 0:
        raise ValueError("element count must be a multiple of 256")
    return out


def num_threads() -> int:
    return int(lib().xo_num_threads())


# ---------------------------------------------------------------- block composition
@dataclass
class MoeWeights:
    """Host copy of one layer's tensors (xabe-engine block/moe.rs:634-658)."""
    num_experts: int
    top_k: int
    hidden: int
    intermediate: int
    eps: float
    post_norm: np.ndarray
    router_f32: np.ndarray | None
    router_q8: np.ndarray | None
    gate_exps: np.ndarray
    up_exps: np.ndarray
    down_exps: np.ndarray
    shared_gate_inp: np.ndarray
    shared_gate: np.ndarray
    shared_up: np.ndarray
    shared_down: np.ndarray
    gate_quant: int = Q6K
    up_quant: int = Q6K
    down_quant: int = Q6K
    sgate_quant: int = Q8_0
    sup_quant: int = Q8_0
    sdown_quant: int = Q8_0


@dataclass
class MoeBlockResult:
    normed: np.ndarray
    logits: np.ndarray
    topk_ids: np.ndarray
    topk_weights: np.ndarray
    routed: np.ndarray
    shexp: np.ndarray
    gate: np.ndarray
    ffn_out: np.ndarray
    l_out: np.ndarray
    seconds_dequant: float
    seconds_matvec: float


def moe_block_forward(w: MoeWeights, residual, logits_override=None, logit_bias=None, threads: int = 1) -> MoeBlockResult:
    x = _f32(residual)
    t, h = x.shape
    assert h == w.hidden
    keep = []  # keep numpy arrays alive for the call

    def f(a):
        if a is None:
            return None
        a = _f32(a)
        keep.append(a)
        return _p(a, _f32p)

    def b(a):
        if a is None:
            return None
        a = _u8(a)
        keep.append(a)
        return _p(a, _u8p)

    cw = _MoeWeights(w.num_experts, w.top_k, w.hidden, w.intermediate, w.eps, f(w.post_norm), f(w.router_f32),
                     b(w.router_q8), w.gate_quant, w.up_quant, w.down_quant, b(w.gate_exps), b(w.up_exps),
                     b(w.down_exps), f(w.shared_gate_inp), w.sgate_quant, w.sup_quant, w.sdown_quant,
                     b(w.shared_gate), b(w.shared_up), b(w.shared_down))
    e, k = w.num_experts, w.top_k
    res = MoeBlockResult(
        normed=np.empty((t, h), np.float32), logits=np.empty((t, e), np.float32),
        topk_ids=np.empty((t, k), np.uint32), topk_weights=np.empty((t, k), np.float32),
        routed=np.empty((t, h), np.float32), shexp=np.empty((t, h), np.float32), gate=np.empty(t, np.float32),
        ffn_out=np.empty((t, h), np.float32), l_out=np.empty((t, h), np.float32), seconds_dequant=0.0,
        seconds_matvec=0.0)
    co = _MoeOutputs(_p(res.normed, _f32p), _p(res.logits, _f32p), _p(res.topk_ids, _u32p),
                     _p(res.topk_weights, _f32p), _p(res.routed, _f32p), _p(res.shexp, _f32p), _p(res.gate, _f32p),
                     _p(res.ffn_out, _f32p), _p(res.l_out, _f32p), 0.0, 0.0)
    rc = lib().xo_moe_block_forward(C.byref(cw), _p(x, _f32p), t, f(logits_override), f(logit_bias), threads,
                                    C.byref(co))
    if rc != 0:
        raise ValueError("moe_block_forward failed")
    res.seconds_dequant = co.seconds_dequant
    res.seconds_matvec = co.seconds_matvec
    return res


def dense_block_forward(hidden: int, intermediate: int, eps: float, post_norm, gate, up, down, residual,
                        quants=(Q6K, Q6K, Q6K), threads: int = 1):
    x = _f32(residual)
    t, h = x.shape
    assert h == hidden
    pn, g, u, d = _f32(post_norm), _u8(gate), _u8(up), _u8(down)
    normed = np.empty((t, h), np.float32)
    ffn_out = np.empty((t, h), np.float32)
    l_out = np.empty((t, h), np.float32)
    rc = lib().xo_dense_block_forward(hidden, intermediate, eps, _p(pn, _f32p), quants[0], quants[1], quants[2],
                                      _p(g, _u8p), _p(u, _u8p), _p(d, _u8p), _p(x, _f32p), t, threads,
                                      _p(normed, _f32p), _p(ffn_out, _f32p), _p(l_out, _f32p))
    if rc != 0:
        raise ValueError("dense_block_forward failed")
    return normed, ffn_out, l_out
