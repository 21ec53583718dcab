"""ctypes binding of the CPU oracle (oracle/moe_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the
benchmark's CPU-baseline leg.  The product package never imports this module.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from dataclasses import dataclass
from typing import Optional

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libmoe_oracle.so")

OK = 0
ERR_DIM = -1
ERR_ZERO_K = -2
ERR_K_EXCEEDS = -3
ERR_NON_FINITE = -4
ERR_NEGATIVE = -5
ERR_SUM_NON_POSITIVE = -6

ATENIA = 0
HUGGINGFACE_QWEN = 1
CERTIFIED = 0  # f64 accumulation (reference default)
STRICT = 1  # f32 accumulation
NORM_GRAPH_F32 = 0  # RmsNorm + BroadcastMul graph nodes, f32 throughout
NORM_F64 = 1  # imperative decoder paths, f64 accumulation


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (seconds).  Returns the .so path."""
    src = os.path.join(_HERE, "moe_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libmoe_oracle.so"],
                              stdout=subprocess.DEVNULL)
    return _SO


class _OraLayer(C.Structure):
    _fields_ = [
        ("num_experts", C.c_int32), ("top_k", C.c_int32), ("d_model", C.c_int32),
        ("d_ff", C.c_int32), ("d_ff_shared", C.c_int32), ("convention", C.c_int32),
        ("w_router", C.c_void_p), ("router_bias", C.c_void_p),
        ("w_gate", C.c_void_p), ("w_up", C.c_void_p), ("w_down", C.c_void_p),
        ("s_gate", C.c_void_p), ("s_up", C.c_void_p), ("s_down", C.c_void_p),
        ("shared_gate", C.c_void_p),
    ]


class _OraV3Config(C.Structure):
    _fields_ = [("n_group", C.c_int32), ("topk_group", C.c_int32), ("norm_topk_prob", C.c_int32),
                ("routed_scaling_factor", C.c_double)]


class _OraMetrics(C.Structure):
    _fields_ = [("max_abs_diff", C.c_double), ("mean_abs_diff", C.c_double),
                ("rmse", C.c_double), ("argmax_match", C.c_int32)]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = C.CDLL(_SO)
        P, Z = C.c_void_p, C.c_size_t
        L.ora_set_threads.argtypes = [C.c_int]
        L.ora_get_threads.restype = C.c_int
        L.ora_hw_threads.restype = C.c_int
        L.ora_f32_to_bf16_bits.argtypes = [C.c_float]
        L.ora_f32_to_bf16_bits.restype = C.c_uint16
        L.ora_bf16_bits_to_f32.argtypes = [C.c_uint16]
        L.ora_bf16_bits_to_f32.restype = C.c_float
        L.ora_seeded.argtypes = [C.c_uint64, Z, P]
        L.ora_silu.argtypes = [C.c_float]
        L.ora_silu.restype = C.c_float
        L.ora_matvec.argtypes = [P, Z, Z, P, P]
        L.ora_matvec_f32acc.argtypes = [P, Z, Z, P, P]
        L.ora_softmax.argtypes = [P, Z, P]
        L.ora_top_k_routing_with.argtypes = [P, Z, Z, C.c_int, P, P, P]
        L.ora_top_k_routing_with.restype = C.c_int
        L.ora_combine_selected.argtypes = [P, P, Z, P, Z, Z, P]
        L.ora_combine_selected.restype = C.c_int
        L.ora_expert_forward.argtypes = [P, P, P, Z, Z, P, P, C.c_int]
        L.ora_sigmoid_dot.argtypes = [P, P, Z]
        L.ora_sigmoid_dot.restype = C.c_float
        L.ora_route.argtypes = [P, P, P, P]
        L.ora_layer_forward_with.argtypes = [P, P, C.c_int, C.c_int, P, P, P, P]
        L.ora_layer_forward_with.restype = C.c_int
        L.ora_execute_layer.argtypes = [P, P, Z, C.c_int, P, P, P, P, P]
        L.ora_execute_layer.restype = C.c_int
        L.ora_rms_norm_gamma.argtypes = [P, P, Z, C.c_float, C.c_int, P]
        L.ora_block_forward.argtypes = [P, P, Z, P, C.c_float, C.c_int, C.c_int, P, P, P, P, P, P]
        L.ora_block_forward.restype = C.c_int
        L.ora_v3_validate.argtypes = [Z, Z, P, P]
        L.ora_v3_validate.restype = C.c_int
        L.ora_v3_route.argtypes = [P, P, Z, Z, P, P, P, P, P, P]
        L.ora_v3_route.restype = C.c_int
        L.ora_v3_layer_forward.argtypes = [P, P, P, P, C.c_int, P, P, P, P]
        L.ora_v3_layer_forward.restype = C.c_int
        L.ora_route_tokens.argtypes = [P, P, Z, P, P, P, P, P]
        L.ora_route_tokens.restype = C.c_int
        L.ora_permute.argtypes = [P, Z, Z, Z, P, P, P]
        L.ora_quantize_per_row_i8.argtypes = [P, Z, Z, P, P]
        L.ora_dequantize_per_row_i8.argtypes = [P, P, Z, Z, P]
        L.ora_absmax_per_channel_symmetric.argtypes = [P, Z, Z, P, P]
        L.ora_int8_to_bf16_per_channel.argtypes = [P, P, Z, Z, P]
        L.ora_absmax_per_group_symmetric.argtypes = [P, Z, Z, Z, P, P]
        L.ora_int8_to_bf16_per_group.argtypes = [P, P, Z, Z, Z, P]
        L.ora_numerical_metrics.argtypes = [P, P, Z, P]
        L.ora_numerical_metrics.restype = C.c_int
        L.ora_layer_forward_f64.argtypes = [P, P, P, P]
        L.ora_layer_forward_f64.restype = C.c_int
        L.ora_expert_forward_f64.argtypes = [P, P, P, Z, Z, P, P]
        _lib = L
    return _lib


def _p(a: Optional[np.ndarray]):
    return None if a is None else a.ctypes.data


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


class OracleError(Exception):
    def __init__(self, rc: int, token: int = -1, index: int = -1):
        self.rc, self.token, self.index = rc, token, index
        super().__init__(f"oracle rc={rc} token={token} index={index}")


def set_threads(n: int) -> None:
    lib().ora_set_threads(int(n))


def hw_threads() -> int:
    return int(lib().ora_hw_threads())


def seeded(seed: int, n: int) -> np.ndarray:
    out = np.empty(n, dtype=np.float32)
    lib().ora_seeded(C.c_uint64(seed), n, _p(out))
    return out


def silu(x: float) -> float:
    return float(lib().ora_silu(C.c_float(x)))


def matvec(w, x, f32acc: bool = False) -> np.ndarray:
    w, x = _f32(w), _f32(x)
    rows, cols = w.shape
    y = np.empty(rows, dtype=np.float32)
    (lib().ora_matvec_f32acc if f32acc else lib().ora_matvec)(_p(w), rows, cols, _p(x), _p(y))
    return y


def softmax(logits) -> np.ndarray:
    logits = _f32(logits)
    out = np.empty_like(logits)
    lib().ora_softmax(_p(logits), logits.size, _p(out))
    return out


def top_k_routing_with(weights, k: int, renormalize: bool = True):
    weights = _f32(weights)
    idx = np.empty(max(k, 1), dtype=np.int32)
    w = np.empty(max(k, 1), dtype=np.float32)
    err = C.c_int32(-1)
    rc = lib().ora_top_k_routing_with(_p(weights), weights.size, k, int(renormalize), _p(idx),
                                      _p(w), C.addressof(err))
    if rc != OK:
        raise OracleError(rc, index=err.value)
    return idx[:k].copy(), w[:k].copy()


def combine_selected(indices, weights, expert_outputs, d_model: int) -> np.ndarray:
    indices = np.ascontiguousarray(indices, dtype=np.int32)
    weights, expert_outputs = _f32(weights), _f32(expert_outputs).reshape(-1)
    out = np.empty(d_model, dtype=np.float32)
    rc = lib().ora_combine_selected(_p(indices), _p(weights), indices.size, _p(expert_outputs),
                                    expert_outputs.size, d_model, _p(out))
    if rc != OK:
        raise OracleError(rc)
    return out


def expert_forward(w_gate, w_up, w_down, x, policy: int = CERTIFIED) -> np.ndarray:
    w_gate, w_up, w_down, x = _f32(w_gate), _f32(w_up), _f32(w_down), _f32(x)
    f, d = w_gate.shape
    y = np.empty(d, dtype=np.float32)
    lib().ora_expert_forward(_p(w_gate), _p(w_up), _p(w_down), d, f, _p(x), _p(y), policy)
    return y


def expert_forward_f64(w_gate, w_up, w_down, x) -> np.ndarray:
    w_gate, w_up, w_down, x = _f32(w_gate), _f32(w_up), _f32(w_down), _f32(x)
    f, d = w_gate.shape
    y = np.empty(d, dtype=np.float64)
    lib().ora_expert_forward_f64(_p(w_gate), _p(w_up), _p(w_down), d, f, _p(x), _p(y))
    return y


def rms_norm_gamma(x, gamma, eps: float, norm_policy: int = 0) -> np.ndarray:
    """RMSNorm(x) * gamma over one row; norm_policy 0 = the graph's f32 arithmetic
    (nn/normalization.rs:8-37 + BroadcastMul), 1 = f64 accumulation (mla.rs:230-239)."""
    x, gamma = _f32(x), _f32(gamma)
    assert x.size == gamma.size
    y = np.empty(x.size, dtype=np.float32)
    lib().ora_rms_norm_gamma(_p(x), _p(gamma), x.size, eps, norm_policy, _p(y))
    return y


V3_ERR_ZERO_PARAMETER, V3_ERR_NOT_DIVISIBLE, V3_ERR_GROUP_TOO_SMALL = -10, -11, -12
V3_ERR_TOPK_GROUP_EXCEEDS, V3_ERR_TOPK_EXCEEDS = -13, -14
V3_ERR_NON_FINITE_LOGIT, V3_ERR_NON_FINITE_BIAS = -15, -16


def v3_route(logits, bias, top_k: int, n_group: int, topk_group: int, scale: float = 1.0,
             norm_topk_prob: bool = True):
    """v3_router.rs:206-309 for one token.  Returns (indices ascending, weights, dense weights,
    selection margin)."""
    logits, bias = _f32(logits), _f32(bias)
    if logits.size != bias.size:
        raise OracleError(ERR_DIM)  # LengthMismatch
    n = logits.size
    cfg = _OraV3Config(n_group, topk_group, int(norm_topk_prob), scale)
    idx = np.empty(max(top_k, 1), dtype=np.int32)
    w = np.empty(max(top_k, 1), dtype=np.float32)
    dense = np.empty(n, dtype=np.float32)
    margin, err = C.c_double(0.0), C.c_int32(-1)
    rc = lib().ora_v3_route(_p(logits), _p(bias), n, top_k, C.addressof(cfg), _p(idx), _p(w),
                            _p(dense), C.addressof(margin), C.addressof(err))
    if rc != OK:
        raise OracleError(rc, index=err.value)
    return idx[:top_k].copy(), w[:top_k].copy(), dense, margin.value


def sigmoid_dot(g, x) -> float:
    g, x = _f32(g), _f32(x)
    return float(lib().ora_sigmoid_dot(_p(g), _p(x), min(g.size, x.size)))


@dataclass
class Layer:
    """Flat-array mirror of the reference's RealMoeLayer (layer.rs:200-212).

    All weights are f32 arrays holding the *stored* values (bf16 / int8
    storage is represented by its exact f32 upcast / dequantisation).
    """
    w_router: np.ndarray  # [E, d]
    w_gate: np.ndarray  # [E, f, d]
    w_up: np.ndarray  # [E, f, d]
    w_down: np.ndarray  # [E, d, f]
    top_k: int
    convention: int = ATENIA
    s_gate: Optional[np.ndarray] = None  # [f_s, d]
    s_up: Optional[np.ndarray] = None
    s_down: Optional[np.ndarray] = None  # [d, f_s]
    shared_gate: Optional[np.ndarray] = None  # [d]
    router_bias: Optional[np.ndarray] = None  # [E] (extension; reference has none)

    def __post_init__(self):
        for n in ("w_router", "w_gate", "w_up", "w_down", "s_gate", "s_up", "s_down",
                  "shared_gate", "router_bias"):
            v = getattr(self, n)
            if v is not None:
                setattr(self, n, _f32(v))
        self.E, self.d = self.w_router.shape
        self.f = self.w_gate.shape[1]
        self.f_s = 0 if self.s_gate is None else self.s_gate.shape[0]
        assert self.w_gate.shape == (self.E, self.f, self.d)
        assert self.w_up.shape == (self.E, self.f, self.d)
        assert self.w_down.shape == (self.E, self.d, self.f)
        if self.shared_gate is not None:
            self.shared_gate = self.shared_gate.reshape(-1)

    def resolve_convention(self) -> int:
        """layer.rs:382-388: gate tensor present => HuggingFaceQwen, else Atenia."""
        return HUGGINGFACE_QWEN if self.shared_gate is not None else ATENIA

    def _c(self, convention: Optional[int] = None) -> _OraLayer:
        return _OraLayer(self.E, self.top_k, self.d, self.f, self.f_s,
                         self.convention if convention is None else convention,
                         _p(self.w_router), _p(self.router_bias), _p(self.w_gate), _p(self.w_up),
                         _p(self.w_down), _p(self.s_gate), _p(self.s_up), _p(self.s_down),
                         _p(self.shared_gate))

    def route(self, x):
        """(logits, softmax weights) of one token."""
        x = _f32(x)
        lo = np.empty(self.E, dtype=np.float32)
        w = np.empty(self.E, dtype=np.float32)
        c = self._c()
        lib().ora_route(C.addressof(c), _p(x), _p(lo), _p(w))
        return lo, w

    def forward_with(self, x, convention: Optional[int] = None, policy: int = CERTIFIED):
        """One token; returns (out[d], idx[k], w[k])."""
        x = _f32(x)
        assert x.size == self.d
        conv = self.convention if convention is None else convention
        out = np.empty(self.d, dtype=np.float32)
        idx = np.empty(max(self.top_k, 1), dtype=np.int32)
        w = np.empty(max(self.top_k, 1), dtype=np.float32)
        err = C.c_int32(-1)
        c = self._c(conv)
        rc = lib().ora_layer_forward_with(C.addressof(c), _p(x), conv, policy, _p(out), _p(idx),
                                          _p(w), C.addressof(err))
        if rc != OK:
            raise OracleError(rc, index=err.value)
        return out, idx[:self.top_k].copy(), w[:self.top_k].copy()

    def execute(self, x, policy: int = CERTIFIED):
        """graph_op.rs:327-350: [T*d] -> [T*d], row by row. Returns (out, idx, w)."""
        x = _f32(x).reshape(-1, self.d)
        T = x.shape[0]
        out = np.empty((T, self.d), dtype=np.float32)
        idx = np.empty((T, self.top_k), dtype=np.int32)
        w = np.empty((T, self.top_k), dtype=np.float32)
        et, ei = C.c_int32(-1), C.c_int32(-1)
        c = self._c()
        rc = lib().ora_execute_layer(C.addressof(c), _p(x), T, policy, _p(out), _p(idx), _p(w),
                                     C.addressof(et), C.addressof(ei))
        if rc != OK:
            raise OracleError(rc, et.value, ei.value)
        return out, idx, w

    def block_forward(self, x1, gamma, eps: float, norm_policy: int = NORM_GRAPH_F32,
                      policy: int = CERTIFIED):
        """full_forward.rs:239-252: out = x1 + MoE(RMSNorm(x1) * gamma), row by row.
        Returns (out, h2, idx, w)."""
        x1 = _f32(x1).reshape(-1, self.d)
        gamma = _f32(gamma)
        assert gamma.size == self.d
        T = x1.shape[0]
        out = np.empty((T, self.d), dtype=np.float32)
        h2 = np.empty((T, self.d), dtype=np.float32)
        idx = np.empty((T, self.top_k), dtype=np.int32)
        w = np.empty((T, self.top_k), dtype=np.float32)
        et, ei = C.c_int32(-1), C.c_int32(-1)
        c = self._c()
        rc = lib().ora_block_forward(C.addressof(c), _p(x1), T, _p(gamma), eps, norm_policy, policy,
                                     _p(out), _p(h2), _p(idx), _p(w), C.addressof(et), C.addressof(ei))
        if rc != OK:
            raise OracleError(rc, et.value, ei.value)
        return out, h2, idx, w

    def v3_forward(self, x, bias, n_group: int, topk_group: int, scale: float, norm_topk_prob: bool,
                   policy: int = CERTIFIED):
        """Rows through the layer with the DeepSeek-V3 router in front (sigmoid scores,
        `bias` = e_score_correction_bias, group-limited top-k, scaled weights), ungated shared
        expert.  Returns (out, idx, w)."""
        x = _f32(x).reshape(-1, self.d)
        bias = _f32(bias)
        assert bias.size == self.E
        T = x.shape[0]
        out = np.empty((T, self.d), dtype=np.float32)
        idx = np.empty((T, self.top_k), dtype=np.int32)
        w = np.empty((T, self.top_k), dtype=np.float32)
        cfg = _OraV3Config(n_group, topk_group, int(norm_topk_prob), scale)
        c = self._c(HUGGINGFACE_QWEN)
        c.shared_gate = None
        for t in range(T):
            err = C.c_int32(-1)
            rc = lib().ora_v3_layer_forward(C.addressof(c), C.addressof(cfg), _p(bias), _p(x[t]),
                                            policy, _p(out[t]), _p(idx[t]), _p(w[t]), C.addressof(err))
            if rc != OK:
                raise OracleError(rc, t, err.value)
        return out, idx, w

    def route_tokens(self, x, want_logits: bool = False):
        x = _f32(x).reshape(-1, self.d)
        T = x.shape[0]
        idx = np.empty((T, self.top_k), dtype=np.int32)
        w = np.empty((T, self.top_k), dtype=np.float32)
        lo = np.empty((T, self.E), dtype=np.float32) if want_logits else None
        et, ei = C.c_int32(-1), C.c_int32(-1)
        c = self._c()
        rc = lib().ora_route_tokens(C.addressof(c), _p(x), T, _p(idx), _p(w), _p(lo),
                                    C.addressof(et), C.addressof(ei))
        if rc != OK:
            raise OracleError(rc, et.value, ei.value)
        return (idx, w, lo) if want_logits else (idx, w)

    def forward_f64(self, x, fixed_idx=None, convention: Optional[int] = None) -> np.ndarray:
        """All-f64 reference of one token."""
        x = _f32(x)
        out = np.empty(self.d, dtype=np.float64)
        fi = None if fixed_idx is None else np.ascontiguousarray(fixed_idx, dtype=np.int32)
        c = self._c(convention)
        rc = lib().ora_layer_forward_f64(C.addressof(c), _p(x), _p(fi), _p(out))
        if rc != OK:
            raise OracleError(rc)
        return out


def permute(idx, num_experts: int):
    """Derived expert-grouping contract: (counts[E], offsets[E+1], perm[T*k])."""
    idx = np.ascontiguousarray(idx, dtype=np.int32)
    T, k = idx.shape
    counts = np.empty(num_experts, dtype=np.int32)
    offsets = np.empty(num_experts + 1, dtype=np.int32)
    perm = np.empty(T * k, dtype=np.int32)
    lib().ora_permute(_p(idx), T, k, num_experts, _p(counts), _p(offsets), _p(perm))
    return counts, offsets, perm


def quantize_per_row_i8(w):
    w = _f32(w)
    rows, cols = w.shape
    q = np.empty((rows, cols), dtype=np.int8)
    s = np.empty(rows, dtype=np.float32)
    lib().ora_quantize_per_row_i8(_p(w), rows, cols, _p(q), _p(s))
    return q, s


def dequantize_per_row_i8(q, scales) -> np.ndarray:
    q = np.ascontiguousarray(q, dtype=np.int8)
    scales = _f32(scales)
    rows, cols = q.shape
    out = np.empty((rows, cols), dtype=np.float32)
    lib().ora_dequantize_per_row_i8(_p(q), _p(scales), rows, cols, _p(out))
    return out


def absmax_per_channel_symmetric(w):
    w = _f32(w)
    k, n = w.shape
    q = np.empty((k, n), dtype=np.int8)
    s = np.empty(n, dtype=np.float32)
    lib().ora_absmax_per_channel_symmetric(_p(w), k, n, _p(q), _p(s))
    return q, s


def int8_to_bf16_per_channel(q, scales) -> np.ndarray:
    q = np.ascontiguousarray(q, dtype=np.int8)
    scales = _f32(scales)
    k, n = q.shape
    out = np.empty((k, n), dtype=np.uint16)
    lib().ora_int8_to_bf16_per_channel(_p(q), _p(scales), k, n, _p(out))
    return out


def absmax_per_group_symmetric(w, group_size: int):
    """quantizer.rs:175-248 on a [K, N] weight: (q [K, N] i8, scales [ceil(K/gs), N])."""
    w = _f32(w)
    k, n = w.shape
    q = np.empty((k, n), dtype=np.int8)
    s = np.empty(((k + group_size - 1) // group_size, n), dtype=np.float32)
    lib().ora_absmax_per_group_symmetric(_p(w), k, n, group_size, _p(q), _p(s))
    return q, s


def int8_to_bf16_per_group(q, scales, group_size: int) -> np.ndarray:
    q = np.ascontiguousarray(q, dtype=np.int8)
    scales = _f32(scales)
    k, n = q.shape
    out = np.empty((k, n), dtype=np.uint16)
    lib().ora_int8_to_bf16_per_group(_p(q), _p(scales), k, n, group_size, _p(out))
    return out


def f32_to_bf16_bits(a) -> np.ndarray:
    """tensor.rs:306-308 truncation, vectorised."""
    return (_f32(a).view(np.uint32) >> 16).astype(np.uint16)


def bf16_bits_to_f32(b) -> np.ndarray:
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def numerical_metrics(a, r) -> dict:
    a, r = _f32(a).reshape(-1), _f32(r).reshape(-1)
    assert a.size == r.size
    m = _OraMetrics()
    rc = lib().ora_numerical_metrics(_p(a), _p(r), a.size, C.addressof(m))
    if rc != OK:
        raise OracleError(rc)
    return dict(max_abs_diff=m.max_abs_diff, mean_abs_diff=m.mean_abs_diff, rmse=m.rmse,
                argmax_match=bool(m.argmax_match))
