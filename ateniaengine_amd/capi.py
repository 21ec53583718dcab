"""ctypes binding of include/atenia_moe_hip.h.

Every call goes to the HIP library; nothing here computes.  Loading fails loudly when the
library has not been built (`make -C ateniaengine_amd/csrc`): there is no CPU fallback.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from typing import Optional

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# ATENIA_MOE_HIP_LIBRARY names another build of the library (same ABI) to load instead.
LIB_PATH = os.environ.get("ATENIA_MOE_HIP_LIBRARY") or os.path.join(_HERE, "libatenia_moe_hip.so")

CONVENTION_ATENIA = 0
CONVENTION_HUGGINGFACE_QWEN = 1
WEIGHT_F32, WEIGHT_BF16, WEIGHT_INT8_W8A16, WEIGHT_INT8_PER_GROUP = 0, 1, 2, 3
ACT_F32, ACT_BF16 = 0, 1
POLICY_CERTIFIED, POLICY_STRICT, POLICY_FAST = 0, 1, 2
KERNELS_STREAM, KERNELS_MID, KERNELS_TILED, KERNELS_F32 = 0, 1, 2, 3
NORM_GRAPH_F32, NORM_F64 = 0, 1
OK, ERR_SYNC, ERR_LAUNCH = 0, 1, 2
ERR_DIM, ERR_K, ERR_NON_FINITE, ERR_OOM, ERR_HANDLE, ERR_UNSUPPORTED = -1, -2, -3, -4, -5, -6
N_STAGES = 6
STAGES = ("router", "permute", "expert_gate_up", "expert_down", "combine", "forward")

# Every symbol include/atenia_moe_hip.h declares.
EXPORTS = (
    "atenia_moe_hip_available", "atenia_moe_hip_last_error_string",
    "atenia_moe_hip_layer_create", "atenia_moe_hip_layer_destroy",
    "atenia_moe_hip_layer_forward", "atenia_moe_hip_layer_forward_device",
    "atenia_moe_hip_layer_status", "atenia_moe_hip_layer_route",
    "atenia_moe_hip_layer_permute", "atenia_moe_hip_layer_last_routing",
    "atenia_moe_hip_layer_last_expert_outputs", "atenia_moe_hip_layer_set_profiling",
    "atenia_moe_hip_layer_stage_ms", "atenia_moe_hip_layer_stage_launches",
    "atenia_moe_hip_layer_info", "atenia_moe_hip_layer_expert_kernels", "atenia_moe_hip_plan_batch", "atenia_moe_hip_layer_last_down_split",
    "atenia_moe_quantize_per_row_i8",
    "atenia_moe_f32_to_bf16_trunc",
    "atenia_moe_hip_layer_last_non_finite", "atenia_moe_router_launch_device", "atenia_moe_permute_launch_device",
    "atenia_moe_expert_ffn_launch_device", "atenia_moe_combine_launch_device",
    "atenia_moe_hip_layer_block_forward", "atenia_moe_hip_layer_block_forward_device",
    "atenia_moe_hip_layer_last_normed", "atenia_moe_hip_layer_set_v3_router",
    "atenia_moe_quantize_per_group_i8",
    "atenia_moe_absmax_per_channel_symmetric", "atenia_moe_absmax_per_group_symmetric",
    "atenia_moe_int8_to_bf16_per_channel_launch_device",
    "atenia_moe_int8_to_bf16_per_group_launch_device",
    "atenia_moe_hip_layer_set_numeric_policy",
    "atenia_moe_hip_layer_forward_device_noalloc",
)
# the reference's own names for the two dequantisation launchers (src/cuda/int8_to_bf16.rs:63-81)
REFERENCE_NAMED_EXPORTS = ("int8_to_bf16_per_channel_launch_device",
                           "int8_to_bf16_per_group_launch_device")


class MoeHipError(RuntimeError):
    def __init__(self, rc: int, msg: str):
        self.rc = rc
        super().__init__(f"atenia_moe_hip rc={rc}: {msg}")


class LayerDesc(C.Structure):
    _fields_ = [
        ("num_experts", C.c_int32), ("top_k", C.c_int32), ("d_model", C.c_int32),
        ("d_ff", C.c_int32), ("d_ff_shared", C.c_int32), ("convention", C.c_int32),
        ("weight_dtype", C.c_int32), ("max_tokens_hint", C.c_int32),
        ("w_router", C.c_void_p), ("router_bias", C.c_void_p),
        ("w_gate", C.c_void_p), ("w_up", C.c_void_p), ("w_down", C.c_void_p),
        ("scale_gate", C.c_void_p), ("scale_up", C.c_void_p), ("scale_down", C.c_void_p),
        ("s_gate", C.c_void_p), ("s_up", C.c_void_p), ("s_down", C.c_void_p),
        ("s_scale_gate", C.c_void_p), ("s_scale_up", C.c_void_p), ("s_scale_down", C.c_void_p),
        ("shared_gate", C.c_void_p), ("group_size", C.c_int32),
    ]


def build(verbose: bool = False) -> str:
    """Compile the HIP library for gfx950 (hipcc cross-compiles without a GPU)."""
    out = None if verbose else subprocess.DEVNULL
    subprocess.check_call(["make", "-C", os.path.join(_HERE, "csrc"), "-B", "-j8"], stdout=out,
                          stderr=out)
    return LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise MoeHipError(ERR_LAUNCH, f"{LIB_PATH} is missing: build it with "
                                          "`make -C ateniaengine_amd/csrc` (no CPU fallback)")
        L = C.CDLL(LIB_PATH)
        P = C.c_void_p
        L.atenia_moe_hip_available.restype = C.c_int
        L.atenia_moe_hip_last_error_string.restype = C.c_char_p
        L.atenia_moe_hip_layer_create.argtypes = [P, P]
        L.atenia_moe_hip_layer_destroy.argtypes = [P]
        L.atenia_moe_hip_layer_forward.argtypes = [P, P, C.c_int, P]
        L.atenia_moe_hip_layer_forward_device.argtypes = [P, P, C.c_int, C.c_int, P, P]
        L.atenia_moe_hip_layer_forward_device_noalloc.argtypes = [P, P, C.c_int, C.c_int, P, P]
        L.atenia_moe_hip_layer_status.argtypes = [P, P, P, P]
        L.atenia_moe_hip_layer_route.argtypes = [P, P, C.c_int, P, P]
        L.atenia_moe_hip_layer_permute.argtypes = [P, P, C.c_int, P, P, P]
        L.atenia_moe_hip_layer_last_routing.argtypes = [P, P, P, P, P, P]
        L.atenia_moe_hip_layer_last_expert_outputs.argtypes = [P, P, P]
        L.atenia_moe_hip_layer_set_profiling.argtypes = [P, C.c_int]
        L.atenia_moe_hip_layer_stage_ms.argtypes = [P, P]
        L.atenia_moe_hip_layer_stage_launches.argtypes = [P, P]
        L.atenia_moe_hip_layer_info.argtypes = [P, P]
        L.atenia_moe_hip_layer_expert_kernels.argtypes = [P, C.c_int64, P]
        L.atenia_moe_hip_plan_batch.argtypes = [C.c_int] * 7 + [C.c_int64, P]
        L.atenia_moe_hip_layer_last_down_split.argtypes = [P, P]
        L.atenia_moe_quantize_per_row_i8.argtypes = [P, C.c_size_t, C.c_size_t, P, P]
        L.atenia_moe_f32_to_bf16_trunc.argtypes = [P, C.c_size_t, P]
        L.atenia_moe_hip_layer_last_non_finite.argtypes = [P, P, P]
        L.atenia_moe_hip_layer_block_forward.argtypes = [P, P, C.c_int, P, C.c_float, C.c_int, P]
        L.atenia_moe_hip_layer_block_forward_device.argtypes = [P, P, C.c_int, P, C.c_float,
                                                                C.c_int, P, P]
        L.atenia_moe_hip_layer_last_normed.argtypes = [P, P]
        L.atenia_moe_quantize_per_group_i8.argtypes = [P, C.c_size_t, C.c_size_t, C.c_size_t, P, P]
        L.atenia_moe_hip_layer_set_v3_router.argtypes = [P, C.c_int, C.c_int, C.c_double, C.c_int, P]
        L.atenia_moe_hip_layer_set_numeric_policy.argtypes = [P, C.c_int]
        L.atenia_moe_absmax_per_channel_symmetric.argtypes = [P, C.c_size_t, C.c_size_t, P, P]
        L.atenia_moe_absmax_per_group_symmetric.argtypes = [P, C.c_size_t, C.c_size_t, C.c_size_t, P, P]
        L.atenia_moe_int8_to_bf16_per_channel_launch_device.argtypes = [P, P, P, C.c_int, C.c_int, P]
        L.atenia_moe_int8_to_bf16_per_group_launch_device.argtypes = [P, P, P, C.c_int, C.c_int,
                                                                      C.c_int, P]
        L.int8_to_bf16_per_channel_launch_device.argtypes = [P, P, P, C.c_int, C.c_int]
        L.int8_to_bf16_per_group_launch_device.argtypes = [P, P, P, C.c_int, C.c_int, C.c_int]
        L.atenia_moe_router_launch_device.argtypes = [P, P, C.c_int, C.c_int, P, P, P]
        L.atenia_moe_permute_launch_device.argtypes = [P, C.c_int, P, P, P, P]
        L.atenia_moe_expert_ffn_launch_device.argtypes = [P, P, C.c_int, C.c_int, P]
        L.atenia_moe_combine_launch_device.argtypes = [P, C.c_int, P, P]
        _lib = L
    return _lib


def _check(rc: int):
    if rc != OK:
        raise MoeHipError(rc, lib().atenia_moe_hip_last_error_string().decode())


def available() -> bool:
    return bool(lib().atenia_moe_hip_available())


def _ptr(a: Optional[np.ndarray]):
    return None if a is None else a.ctypes.data


def _arr(a, dtype):
    return None if a is None else np.ascontiguousarray(a, dtype=dtype)


def quantize_per_row_i8(w):
    w = np.ascontiguousarray(w, dtype=np.float32)
    rows = int(np.prod(w.shape[:-1]))
    cols = w.shape[-1]
    q = np.empty(w.shape, dtype=np.int8)
    s = np.empty(w.shape[:-1], dtype=np.float32)
    _check(lib().atenia_moe_quantize_per_row_i8(_ptr(w), rows, cols, _ptr(q), _ptr(s)))
    return q, s


def quantize_per_group_i8(w, group_size: int):
    """Per-group symmetric int8 along the last axis: returns (q like w, scales [..., ceil(cols/gs)])."""
    w = np.ascontiguousarray(w, dtype=np.float32)
    rows = int(np.prod(w.shape[:-1]))
    cols = w.shape[-1]
    q = np.empty(w.shape, dtype=np.int8)
    s = np.empty(w.shape[:-1] + ((cols + group_size - 1) // group_size,), dtype=np.float32)
    _check(lib().atenia_moe_quantize_per_group_i8(_ptr(w), rows, cols, group_size, _ptr(q), _ptr(s)))
    return q, s


def absmax_per_channel_symmetric(w):
    """[K, N] weight -> (q [K, N] int8, scales [N]), one scale per column
    (src/tensor/quantizer.rs:67-117)."""
    w = np.ascontiguousarray(w, dtype=np.float32)
    k, n = w.shape
    q = np.empty((k, n), dtype=np.int8)
    s = np.empty(n, dtype=np.float32)
    _check(lib().atenia_moe_absmax_per_channel_symmetric(_ptr(w), k, n, _ptr(q), _ptr(s)))
    return q, s


def absmax_per_group_symmetric(w, group_size: int):
    """[K, N] weight -> (q [K, N] int8, scales [ceil(K/gs), N]), groups along K
    (src/tensor/quantizer.rs:175-248)."""
    w = np.ascontiguousarray(w, dtype=np.float32)
    k, n = w.shape
    q = np.empty((k, n), dtype=np.int8)
    s = np.empty(((k + group_size - 1) // group_size, n), dtype=np.float32)
    _check(lib().atenia_moe_absmax_per_group_symmetric(_ptr(w), k, n, group_size, _ptr(q), _ptr(s)))
    return q, s


def int8_to_bf16_launch_device(d_int8, d_scales, d_bf16, k: int, n: int, group_size: int = 0,
                               stream=None, reference_symbol: bool = False) -> int:
    """Launches the device dequantisation of a [K, N] int8 weight (device pointers as ints);
    group_size 0 = one scale per column.  Returns the launcher's status code unchanged, as the
    reference's wrapper receives it (src/cuda/int8_to_bf16.rs).  `reference_symbol` goes through
    the entry points that carry the reference's own names (default stream)."""
    L = lib()
    if reference_symbol:
        if group_size:
            return L.int8_to_bf16_per_group_launch_device(d_int8, d_scales, d_bf16, k, n, group_size)
        return L.int8_to_bf16_per_channel_launch_device(d_int8, d_scales, d_bf16, k, n)
    if group_size:
        return L.atenia_moe_int8_to_bf16_per_group_launch_device(d_int8, d_scales, d_bf16, k, n,
                                                                 group_size, stream)
    return L.atenia_moe_int8_to_bf16_per_channel_launch_device(d_int8, d_scales, d_bf16, k, n, stream)


PLAN_KEYS = ("up", "down", "shared_up", "shared_down", "y_bf16", "ys_bf16", "tall_tiles", "duo")


def plan_batch(E: int, k: int, d: int, f: int, f_s: int, weight_dtype: int, T: int,
               group_size: int = 0) -> dict:
    """Which kernels a T-token batch takes on a layer of these dimensions (no device needed):
    kernel family per phase for the routed and the shared expert (KERNELS_*; -1 = none), whether
    the expert outputs reach the combine as bf16, tall row tiles, two-workgroup form per phase
    (`duo`, bits 0 and 1), and `int8_copy`: a W8A16 layer's tiled phases on the bf16 copy of its
    int8 values."""
    v = np.zeros(8, dtype=np.int32)
    _check(lib().atenia_moe_hip_plan_batch(E, k, d, f, f_s, weight_dtype, group_size, T, _ptr(v)))
    plan = dict(zip(PLAN_KEYS, (int(i) for i in v)))
    plan["int8_copy"] = (plan["duo"] >> 2) & 1
    plan["duo"] &= 3
    return plan


def f32_to_bf16_trunc(a) -> np.ndarray:
    a = np.ascontiguousarray(a, dtype=np.float32)
    out = np.empty(a.shape, dtype=np.uint16)
    _check(lib().atenia_moe_f32_to_bf16_trunc(_ptr(a), a.size, _ptr(out)))
    return out


_WDTYPE_NP = {WEIGHT_F32: np.float32, WEIGHT_BF16: np.uint16, WEIGHT_INT8_W8A16: np.int8,
              WEIGHT_INT8_PER_GROUP: np.int8}


class Layer:
    """Owns one `AteniaMoeLayer*`."""

    def __init__(self, *, w_router, w_gate, w_down, top_k, w_up=None, convention=CONVENTION_ATENIA,
                 weight_dtype=WEIGHT_F32, router_bias=None, scale_gate=None, scale_up=None,
                 scale_down=None, s_gate=None, s_up=None, s_down=None, s_scale_gate=None,
                 s_scale_up=None, s_scale_down=None, shared_gate=None, max_tokens_hint=0,
                 group_size=0):
        wt = _WDTYPE_NP[weight_dtype]
        w_router = _arr(w_router, np.float32)
        E, d = w_router.shape
        w_gate, w_up, w_down = _arr(w_gate, wt), _arr(w_up, wt), _arr(w_down, wt)
        f = w_down.shape[2]
        if w_up is None:
            assert w_gate.shape == (E, 2 * f, d), "packed gate_up must be [E, 2f, d]"
        else:
            assert w_gate.shape == (E, f, d) and w_up.shape == (E, f, d)
        assert w_down.shape == (E, d, f)
        s_gate, s_up, s_down = _arr(s_gate, wt), _arr(s_up, wt), _arr(s_down, wt)
        fs = 0 if s_gate is None else s_gate.shape[0]
        keep = dict(
            w_router=w_router, router_bias=_arr(router_bias, np.float32), w_gate=w_gate, w_up=w_up,
            w_down=w_down, scale_gate=_arr(scale_gate, np.float32),
            scale_up=_arr(scale_up, np.float32), scale_down=_arr(scale_down, np.float32),
            s_gate=s_gate, s_up=s_up, s_down=s_down, s_scale_gate=_arr(s_scale_gate, np.float32),
            s_scale_up=_arr(s_scale_up, np.float32), s_scale_down=_arr(s_scale_down, np.float32),
            shared_gate=None if shared_gate is None else _arr(shared_gate, np.float32).reshape(-1))
        desc = LayerDesc(E, top_k, d, f, fs, convention, weight_dtype, max_tokens_hint,
                         *[_ptr(keep[n]) for n in (
                             "w_router", "router_bias", "w_gate", "w_up", "w_down", "scale_gate",
                             "scale_up", "scale_down", "s_gate", "s_up", "s_down", "s_scale_gate",
                             "s_scale_up", "s_scale_down", "shared_gate")], group_size)
        self.E, self.k, self.d, self.f, self.fs = E, top_k, d, f, fs
        self.convention, self.weight_dtype, self.group_size = convention, weight_dtype, group_size
        self._h = C.c_void_p()
        _check(lib().atenia_moe_hip_layer_create(C.addressof(desc), C.addressof(self._h)))
        del keep  # host arrays are only borrowed for the call

    def close(self):
        if getattr(self, "_h", None) is not None and self._h.value:
            lib().atenia_moe_hip_layer_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.close()

    # -- the op ---------------------------------------------------------------------------
    def forward(self, x, out=None) -> np.ndarray:
        """[T, d] (or [T*d]) f32 host -> same shape f32 host (into `out` when given)."""
        x = np.ascontiguousarray(x, dtype=np.float32)
        assert x.size % self.d == 0
        if out is None:
            out = np.empty_like(x)
        assert out.dtype == np.float32 and out.size == x.size and out.flags.c_contiguous
        _check(lib().atenia_moe_hip_layer_forward(self._h, _ptr(x), x.size // self.d, _ptr(out)))
        return out

    def forward_device(self, d_x: int, x_dtype: int, n_tokens: int, d_out: int, stream: int = 0):
        """Raw device pointers (ints); asynchronous on `stream`."""
        _check(lib().atenia_moe_hip_layer_forward_device(self._h, d_x, x_dtype, n_tokens, d_out,
                                                         stream))

    def forward_device_noalloc(self, d_x: int, x_dtype: int, n_tokens: int, d_out: int,
                               stream: int = 0):
        """forward_device on the library's static workspace: the call allocates nothing."""
        _check(lib().atenia_moe_hip_layer_forward_device_noalloc(self._h, d_x, x_dtype, n_tokens,
                                                                 d_out, stream))

    def set_v3_router(self, n_group: int, topk_group: int, routed_scaling_factor: float,
                      norm_topk_prob: bool, e_score_correction_bias):
        """DeepSeek-V3 routing for every later call on this layer (v3_router.rs:206-309)."""
        b = np.ascontiguousarray(e_score_correction_bias, dtype=np.float32)
        assert b.size == self.E
        _check(lib().atenia_moe_hip_layer_set_v3_router(self._h, n_group, topk_group,
                                                        routed_scaling_factor, int(norm_topk_prob),
                                                        _ptr(b)))

    def set_numeric_policy(self, policy: int):
        """Expert arithmetic of an f32 layer from the next forward on: POLICY_CERTIFIED (f64
        accumulation), POLICY_STRICT / POLICY_FAST (f32 accumulation); numeric_policy.rs:36-75."""
        _check(lib().atenia_moe_hip_layer_set_numeric_policy(self._h, policy))

    # The decoder layer's FFN block around the op: out = x1 + MoE(RMSNorm(x1) * gamma).
    def block_forward(self, x1, gamma, eps: float, norm_policy: int = NORM_GRAPH_F32) -> np.ndarray:
        x1 = np.ascontiguousarray(x1, dtype=np.float32)
        gamma = np.ascontiguousarray(gamma, dtype=np.float32)
        assert x1.size % self.d == 0 and gamma.size == self.d
        out = np.empty_like(x1)
        _check(lib().atenia_moe_hip_layer_block_forward(self._h, _ptr(x1), x1.size // self.d,
                                                        _ptr(gamma), eps, norm_policy, _ptr(out)))
        return out

    def block_forward_device(self, d_x1: int, n_tokens: int, d_gamma: int, eps: float,
                             norm_policy: int, d_out: int, stream: int = 0):
        _check(lib().atenia_moe_hip_layer_block_forward_device(self._h, d_x1, n_tokens, d_gamma, eps,
                                                               norm_policy, d_out, stream))

    def last_normed(self, T: int) -> np.ndarray:
        h2 = np.empty((T, self.d), dtype=np.float32)
        _check(lib().atenia_moe_hip_layer_last_normed(self._h, _ptr(h2)))
        return h2

    # Stage launchers: the pipeline one kernel at a time (raw device pointers as ints, 0 = NULL).
    def router_device(self, d_x: int, x_dtype: int, n_tokens: int, d_idx: int = 0, d_w: int = 0,
                      stream: int = 0):
        _check(lib().atenia_moe_router_launch_device(self._h, d_x, x_dtype, n_tokens, d_idx or None,
                                                     d_w or None, stream))

    def permute_device(self, n_tokens: int, d_counts: int = 0, d_offsets: int = 0, d_perm: int = 0,
                       stream: int = 0):
        _check(lib().atenia_moe_permute_launch_device(self._h, n_tokens, d_counts or None,
                                                      d_offsets or None, d_perm or None, stream))

    def expert_ffn_device(self, d_x: int, x_dtype: int, n_tokens: int, stream: int = 0):
        _check(lib().atenia_moe_expert_ffn_launch_device(self._h, d_x, x_dtype, n_tokens, stream))

    def combine_device(self, n_tokens: int, d_out: int, stream: int = 0):
        _check(lib().atenia_moe_combine_launch_device(self._h, n_tokens, d_out, stream))

    def status(self, stream: int = 0):
        tok, ex = C.c_int32(-1), C.c_int32(-1)
        rc = lib().atenia_moe_hip_layer_status(self._h, stream, C.addressof(tok), C.addressof(ex))
        return rc, tok.value, ex.value

    def last_non_finite(self):
        """(token, expert) of the most recent non-finite routing weight, (-1, -1) if none."""
        tok, ex = C.c_int32(-1), C.c_int32(-1)
        _check(lib().atenia_moe_hip_layer_last_non_finite(self._h, C.addressof(tok), C.addressof(ex)))
        return tok.value, ex.value

    # -- parity taps ----------------------------------------------------------------------
    def route(self, x):
        x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, self.d)
        T = x.shape[0]
        idx = np.empty((T, self.k), dtype=np.int32)
        w = np.empty((T, self.k), dtype=np.float32)
        _check(lib().atenia_moe_hip_layer_route(self._h, _ptr(x), T, _ptr(idx), _ptr(w)))
        return idx, w

    def permute(self, idx):
        idx = np.ascontiguousarray(idx, dtype=np.int32).reshape(-1, self.k)
        T = idx.shape[0]
        counts = np.empty(self.E, dtype=np.int32)
        offsets = np.empty(self.E + 1, dtype=np.int32)
        perm = np.empty(T * self.k, dtype=np.int32)
        _check(lib().atenia_moe_hip_layer_permute(self._h, _ptr(idx), T, _ptr(counts),
                                                  _ptr(offsets), _ptr(perm)))
        return counts, offsets, perm

    def last_routing(self, T: int):
        idx = np.empty((T, self.k), dtype=np.int32)
        w = np.empty((T, self.k), dtype=np.float32)
        counts = np.empty(self.E, dtype=np.int32)
        offsets = np.empty(self.E + 1, dtype=np.int32)
        perm = np.empty(T * self.k, dtype=np.int32)
        _check(lib().atenia_moe_hip_layer_last_routing(self._h, _ptr(idx), _ptr(w), _ptr(counts),
                                                       _ptr(offsets), _ptr(perm)))
        return idx, w, counts, offsets, perm

    def last_expert_outputs(self, T: int):
        y = np.empty((T, self.k, self.d), dtype=np.float32)
        ys = np.empty((T, self.d), dtype=np.float32) if self.fs else None
        _check(lib().atenia_moe_hip_layer_last_expert_outputs(self._h, _ptr(y), _ptr(ys)))
        return y, ys

    def last_down_split(self, T: int) -> np.ndarray:
        """[T, k, ceil(d / 256)] k ranges of the down tile behind each expert-output block (1 = whole)."""
        parts = np.empty((T, self.k, (self.d + 255) // 256), dtype=np.uint8)
        _check(lib().atenia_moe_hip_layer_last_down_split(self._h, _ptr(parts)))
        return parts

    # -- timing ---------------------------------------------------------------------------
    def set_profiling(self, on: bool):
        _check(lib().atenia_moe_hip_layer_set_profiling(self._h, int(on)))

    def stage_ms(self) -> np.ndarray:
        ms = np.zeros(N_STAGES, dtype=np.float32)
        _check(lib().atenia_moe_hip_layer_stage_ms(self._h, _ptr(ms)))
        return ms

    def stage_launches(self) -> np.ndarray:
        n = np.zeros(N_STAGES, dtype=np.int32)
        _check(lib().atenia_moe_hip_layer_stage_launches(self._h, _ptr(n)))
        return n

    def expert_kernels(self, T: int):
        """(routed, shared) kernel family a batch of T tokens takes: KERNELS_STREAM / _MID /
        _TILED / _F32; shared is -1 for a layer without a shared expert."""
        v = np.zeros(2, dtype=np.int32)
        _check(lib().atenia_moe_hip_layer_expert_kernels(self._h, T, _ptr(v)))
        return int(v[0]), int(v[1])

    def plan(self, T: int) -> dict:
        """plan_batch for this layer's dimensions."""
        return plan_batch(self.E, self.k, self.d, self.f, self.fs, self.weight_dtype, T,
                          self.group_size)

    def info(self) -> dict:
        v = np.zeros(8, dtype=np.int64)
        _check(lib().atenia_moe_hip_layer_info(self._h, _ptr(v)))
        keys = ("E", "k", "d", "f", "f_s", "convention", "weight_dtype", "bytes_per_expert")
        return dict(zip(keys, (int(i) for i in v)))
