"""CPU-side checks of the C-ABI library: it loads, exports every symbol the header declares,
and its host-only helpers (no GPU involved) match the oracle bit for bit."""
import os
import re

import numpy as np

from ateniaengine_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "atenia_moe_hip.h")).read()
    declared = set(re.findall(r"\b(atenia_moe_\w+)\s*\(", header))
    assert declared == set(capi.EXPORTS)
    L = capi.lib()
    for name in declared:
        assert hasattr(L, name), f"{name} is declared but not exported"
    # the two dequantisation launchers that keep the reference's symbol names
    plain = set(re.findall(r"^int (int8_to_bf16_\w+)\s*\(", header, flags=re.M))
    assert plain == set(capi.REFERENCE_NAMED_EXPORTS)
    for name in plain:
        assert hasattr(L, name), f"{name} is declared but not exported"


def test_last_error_string_and_bad_handles():
    L = capi.lib()
    assert L.atenia_moe_hip_layer_destroy(None) == capi.ERR_HANDLE
    assert b"invalid layer handle" in L.atenia_moe_hip_last_error_string()
    assert L.atenia_moe_hip_layer_forward(None, None, 1, None) == capi.ERR_HANDLE
    assert L.atenia_moe_hip_layer_create(None, None) == capi.ERR_DIM


def test_host_quantiser_matches_oracle(ora):
    rng = np.random.default_rng(0)
    w = (rng.standard_normal((64, 129)) * 0.02).astype(np.float32)
    w[5] = 0
    w[7] *= 8
    q, s = capi.quantize_per_row_i8(w)
    oq, os_ = ora.quantize_per_row_i8(w)
    assert (q == oq).all() and s.tobytes() == os_.tobytes()


def test_host_kn_quantisers_match_oracle(ora):
    """[K, N]-oriented quantisers (src/tensor/quantizer.rs:67-117, 175-248) against the oracle,
    with an all-zero column, an outlier and a ragged last group."""
    rng = np.random.default_rng(2)
    w = (rng.standard_normal((200, 37)) * 0.02).astype(np.float32)
    w[:, 3] = 0
    w[17, 5] *= 40
    q, s = capi.absmax_per_channel_symmetric(w)
    oq, os_ = ora.absmax_per_channel_symmetric(w)
    assert (q == oq).all() and s.tobytes() == os_.tobytes()
    for gs in (1, 64, 128, 200, 512):
        q, s = capi.absmax_per_group_symmetric(w, gs)
        oq, os_ = ora.absmax_per_group_symmetric(w, gs)
        assert (q == oq).all() and s.tobytes() == os_.tobytes(), gs
    # the known-answer case of the reference's own test (quantizer.rs:969-993)
    q, s = capi.absmax_per_channel_symmetric(np.array([[2.0], [-4.0], [6.0], [-127.0]], np.float32))
    assert s.tolist() == [1.0] and q.reshape(-1).tolist() == [2, -4, 6, -127]


def test_dequant_launchers_check_their_arguments():
    """Argument checks run before anything touches the GPU: empty shapes are a no-op (0), a
    non-positive group size is -2 (src/cuda/int8_to_bf16.cu:57-59, 122), null pointers -1."""
    assert capi.int8_to_bf16_launch_device(None, None, None, 0, 16) == 0
    assert capi.int8_to_bf16_launch_device(None, None, None, 16, 0, group_size=8) == 0
    L = capi.lib()
    assert L.atenia_moe_int8_to_bf16_per_group_launch_device(None, None, None, 4, 4, 0, None) == -2
    assert L.int8_to_bf16_per_group_launch_device(None, None, None, 4, 4, -1) == -2
    assert capi.int8_to_bf16_launch_device(None, None, None, 4, 4) == -1
    assert capi.int8_to_bf16_launch_device(None, None, None, 4, 4, reference_symbol=True) == -1


def test_host_bf16_truncation_matches_oracle(ora):
    a = np.random.default_rng(1).standard_normal(4097).astype(np.float32)
    assert (capi.f32_to_bf16_trunc(a) == ora.f32_to_bf16_bits(a)).all()


def test_missing_gpu_fails_loudly():
    """Without a GPU the product path refuses to run; it never computes on the CPU."""
    if capi.available():
        return
    import pytest
    with pytest.raises(capi.MoeHipError) as e:
        capi.Layer(w_router=np.zeros((2, 4), np.float32), w_gate=np.zeros((2, 4, 4), np.float32),
                   w_up=np.zeros((2, 4, 4), np.float32), w_down=np.zeros((2, 4, 4), np.float32),
                   top_k=1)
    assert e.value.rc == capi.ERR_LAUNCH and "no gfx950 device" in str(e.value)
