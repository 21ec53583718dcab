"""Seeded random layer shapes through the whole pipeline: expert counts from 1 to 70, any top-k,
widths that are not multiples of the kernels' tile sizes, batch sizes on both sides of every
kernel-selection threshold, all three storage types and both conventions.  Same bars as the
fixed cases of test_gpu_parity.py (routing and grouping bit-exact, outputs within tolerance, and
within 1e-3 of the NumPy model of the blocked kernels' arithmetic)."""
import numpy as np
import pytest

from ateniaengine_amd import capi
from tests import synth as S
from tests.test_gpu_parity import TOL_BF16_TOY, TOL_F32, check_layer

pytestmark = pytest.mark.gpu


def _cases(n, seed):
    rng = np.random.default_rng(seed)
    out = []
    for i in range(n):
        E = int(rng.choice([1, 2, 3, 5, 8, 17, 33, 60, 64, 65, 70]))
        k = int(rng.integers(1, min(E, 8) + 1))
        d = int(rng.choice([8, 24, 37, 64, 100, 128, 200, 256, 320]))
        f = int(rng.choice([8, 20, 33, 64, 96, 130, 256, 400]))
        shared = bool(rng.integers(0, 2))
        fs = int(rng.choice([16, 50, 128, 272])) if shared else 0
        gated = shared and bool(rng.integers(0, 2))
        conv = int(rng.integers(0, 2)) if shared else 0
        wd = [capi.WEIGHT_F32, capi.WEIGHT_BF16, capi.WEIGHT_INT8_W8A16][i % 3]
        T = int(rng.choice([1, 2, 3, 15, 16, 17, 31, 32, 33, 47, 48, 49, 63, 64, 65, 127, 128, 129,
                            255, 256, 257, 300, 511, 513, 800, 1100]))
        if wd == capi.WEIGHT_F32:
            T = min(T, 130)  # the f32 path is the slow one on both sides
        out.append(pytest.param(E, k, d, f, fs, gated, conv, wd, T, 1000 + i,
                                id=f"{i}-E{E}k{k}d{d}f{f}s{fs}g{int(gated)}c{conv}w{wd}T{T}"))
    return out


@pytest.mark.parametrize("E,k,d,f,fs,gated,conv,wd,T,seed", _cases(150, 20240607))
def test_random_layer(ora, E, k, d, f, fs, gated, conv, wd, T, seed):
    W = S.make_weights(seed, E, d, f, f_s=fs, gated=gated, router_std=1.0 / np.sqrt(d),
                       outlier_frac=0.01 if wd == capi.WEIGHT_INT8_W8A16 else 0.0)
    oL, gL = S.build_pair(ora, W, k, conv, wd)
    with gL:
        x = S.make_tokens(seed + 1, T, d, bf16=wd != capi.WEIGHT_F32)
        tol = TOL_F32 if wd == capi.WEIGHT_F32 else TOL_BF16_TOY
        sample = None if T <= 64 else sorted(set(np.linspace(0, T - 1, 48).astype(int).tolist()))
        check_layer(ora, oL, gL, x, tol, sample=sample)
        # a second, smaller batch on the same handle (grow-only workspace, stale state)
        T2 = max(1, T // 3)
        check_layer(ora, oL, gL, x[:T2], tol, sample=None if T2 <= 64 else range(0, T2, max(1, T2 // 40)))


def _mid_cases(n, seed):
    """Shapes the mid-batch kernel can take (K in whole 64-k / 128-k stages) at batch sizes inside
    and on both sides of its bounds, with and without a shared expert it can take along."""
    rng = np.random.default_rng(seed)
    out = []
    for i in range(n):
        wd = [capi.WEIGHT_BF16, capi.WEIGHT_INT8_W8A16][i % 2]
        step = 128 if wd == capi.WEIGHT_INT8_W8A16 else 64
        E = int(rng.choice([2, 4, 8, 16, 60]))
        k = int(rng.integers(1, min(E, 6) + 1))
        d = step * int(rng.integers(1, 4))
        f = step * int(rng.integers(1, 6))
        shared = bool(rng.integers(0, 2))
        fs = (step * int(rng.integers(1, 9)) if rng.integers(0, 4) else 72) if shared else 0
        gated = shared and bool(rng.integers(0, 2))
        conv = int(rng.integers(0, 2)) if shared else 0
        rows = float(rng.choice([3, 8, 14, 20, 35, 50, 70, 100, 130]))  # per expert on average
        T = int(min(900, max(20, round(rows * E / k + rng.integers(-2, 3)))))
        out.append(pytest.param(E, k, d, f, fs, gated, conv, wd, T, 3000 + i,
                                id=f"{i}-E{E}k{k}d{d}f{f}s{fs}g{int(gated)}c{conv}w{wd}T{T}"))
    return out


_MID_SEEN = []


@pytest.mark.parametrize("E,k,d,f,fs,gated,conv,wd,T,seed", _mid_cases(60, 20250311))
def test_random_layer_mid_batch(ora, E, k, d, f, fs, gated, conv, wd, T, seed):
    W = S.make_weights(seed, E, d, f, f_s=fs, gated=gated, router_std=1.0 / np.sqrt(d),
                       outlier_frac=0.01 if wd == capi.WEIGHT_INT8_W8A16 else 0.0)
    oL, gL = S.build_pair(ora, W, k, conv, wd)
    with gL:
        _MID_SEEN.append(gL.expert_kernels(T))
        x = S.make_tokens(seed + 1, T, d)
        sample = None if T <= 64 else sorted(set(np.linspace(0, T - 1, 48).astype(int).tolist()))
        check_layer(ora, oL, gL, x, TOL_BF16_TOY, sample=sample)


def test_random_layer_mid_batch_reached_the_kernel():
    """The cases above must have exercised the mid-batch family, alone and with a shared expert
    inside its launches (this runs after them: same module, defined later)."""
    if len(_MID_SEEN) != 60:
        pytest.skip("needs the 60 cases above to have run in this process")
    routed_mid = sum(1 for r, s in _MID_SEEN if r == capi.KERNELS_MID)
    shared_mid = sum(1 for r, s in _MID_SEEN if r == capi.KERNELS_MID and s == capi.KERNELS_MID)
    assert routed_mid >= 20 and shared_mid >= 5, (routed_mid, shared_mid)


def _router_cases(n, seed):
    """bf16 activations on the device with router rows that fit bf16: every form of the router on
    the f64 matrix cores (rows dealt to workgroups or not, one to five row blocks, more than 64
    experts) and the per-token kernel below their batch sizes."""
    rng = np.random.default_rng(seed)
    out = []
    for i in range(n):
        E = int(rng.choice([2, 8, 15, 16, 17, 31, 32, 33, 48, 60, 64, 65, 79, 80, 96, 128, 200, 255]))
        k = int(rng.integers(1, min(E, 8) + 1))
        d = int(rng.choice([8, 64, 96, 256, 520, 1024, 2048]))
        T = int(rng.choice([2, 17, 51, 52, 53, 191, 192, 193, 300, 511, 513, 1000, 2048, 2049, 3000]))
        gated = bool(rng.integers(0, 2)) and E < 255
        bias = bool(rng.integers(0, 2))
        wide = bool(rng.integers(0, 3) == 0)  # activations over 60 binades: sequential fallback
        out.append(pytest.param(E, k, d, T, gated, bias, wide, 3000 + i,
                                id=f"{i}-E{E}k{k}d{d}T{T}g{int(gated)}b{int(bias)}w{int(wide)}"))
    return out


@pytest.mark.parametrize("E,k,d,T,gated,bias,wide,seed", _router_cases(60, 20251125))
def test_random_router_on_device_bf16(ora, E, k, d, T, gated, bias, wide, seed):
    from tests.hipmem import DeviceArray
    from tests.test_gpu_parity import ulp_diff
    b = -1.2 * np.log(np.random.default_rng(seed).permutation(E) + 1.0) if bias else None
    W = S.make_weights(seed, E, d, 16, f_s=16 if gated else 0, gated=gated,
                       router_std=1.0 / np.sqrt(d), bias=b)
    W["w_router"] = S.bf16_round_trip(W["w_router"])[1]
    if gated:
        W["shared_gate"] = S.bf16_round_trip(W["shared_gate"])[1]
    conv = capi.CONVENTION_HUGGINGFACE_QWEN if gated else capi.CONVENTION_ATENIA
    oL, gL = S.build_pair(ora, W, k, conv, capi.WEIGHT_BF16)
    rng = np.random.default_rng(seed + 1)
    if wide:
        x = rng.standard_normal((T, d)) * np.exp2(rng.integers(-30, 30, size=(T, d)))
    else:
        x = rng.standard_normal((T, d))
    x = S.bf16_round_trip(x.astype(np.float32))[1]
    bits = (x.view(np.uint32) >> 16).astype(np.uint16)
    with gL:
        dx = DeviceArray.from_host(bits)
        out = DeviceArray((T, d), np.float32, fill=0)
        gL.forward_device(dx.ptr, capi.ACT_BF16, T, out.ptr)
        idx, w, counts, offsets, perm = gL.last_routing(T)
        o_idx, o_w = oL.route_tokens(x)
        assert (idx == o_idx).all(), f"{(idx != o_idx).any(axis=1).sum()} tokens routed differently"
        assert ulp_diff(w, o_w).max() <= 1
        oc, oo, op = ora.permute(o_idx, E)
        assert (counts == oc).all() and (offsets == oo).all() and (perm == op).all()
