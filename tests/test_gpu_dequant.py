"""INT8 -> BF16 dequantisation launchers (src/cuda/int8_to_bf16.cu:24-71, 91-141) against the
oracle's restatement, bit for bit: per channel and per group, through the stream-taking entry
points and through the ones that keep the reference's symbol names, on the vector kernel (rows of
a multiple of 8 elements, aligned pointers) and on the one-element kernel (everything else)."""
import numpy as np
import pytest

from ateniaengine_amd import capi
from tests.hipmem import DeviceArray, Stream, hip

pytestmark = pytest.mark.gpu


def _weights(seed, k, n):
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((k, n)) * 0.02).astype(np.float32)
    if n > 3:
        w[:, 3] = 0.0                                   # all-zero column -> the 1e-12 floor
    w[rng.integers(0, k), rng.integers(0, n)] *= 50.0   # an outlier
    return w


def _run(q, s, k, n, gs, stream=None, reference_symbol=False, offset=0):
    """Dequantises on the device; `offset` shifts the int8 pointer off 16-byte alignment."""
    pad = np.zeros(offset, np.int8)
    dq = DeviceArray.from_host(np.concatenate([pad, q.reshape(-1)]))
    ds = DeviceArray.from_host(s)
    dout = DeviceArray((k, n), np.uint16, fill=0xEE)
    rc = capi.int8_to_bf16_launch_device(dq.ptr + offset, ds.ptr, dout.ptr, k, n, group_size=gs,
                                         stream=stream.ptr if stream else None,
                                         reference_symbol=reference_symbol)
    assert rc == 0, rc
    if stream:
        stream.synchronize()
    return dout.to_host()


SHAPES = [(64, 128), (129, 8), (1, 8), (200, 37), (7, 1), (33, 1000), (512, 4096), (1500, 1408)]


@pytest.mark.parametrize("k,n", SHAPES)
def test_per_channel_matches_oracle(ora, k, n):
    q, s = capi.absmax_per_channel_symmetric(_weights(k * 31 + n, k, n))
    q[0, 0] = -128                                      # not produced by the quantiser, still legal int8
    want = ora.int8_to_bf16_per_channel(q, s)
    stream = Stream()
    assert _run(q, s, k, n, 0, stream=stream).tobytes() == want.tobytes()
    assert _run(q, s, k, n, 0, reference_symbol=True).tobytes() == want.tobytes()
    stream.close()


@pytest.mark.parametrize("k,n", SHAPES)
@pytest.mark.parametrize("gs", [128, 64, 7, 4096])
def test_per_group_matches_oracle(ora, k, n, gs):
    q, s = capi.absmax_per_group_symmetric(_weights(k * 17 + n + gs, k, n), gs)
    assert s.shape == ((k + gs - 1) // gs, n)
    want = ora.int8_to_bf16_per_group(q, s, gs)
    stream = Stream()
    assert _run(q, s, k, n, gs, stream=stream).tobytes() == want.tobytes()
    assert _run(q, s, k, n, gs, reference_symbol=True).tobytes() == want.tobytes()
    stream.close()


def test_unaligned_pointer_takes_the_element_kernel(ora):
    k, n = 96, 256
    q, s = capi.absmax_per_group_symmetric(_weights(5, k, n), 32)
    want = ora.int8_to_bf16_per_group(q, s, 32)
    for off in (1, 8):
        assert _run(q, s, k, n, 32, offset=off).tobytes() == want.tobytes(), off


def test_signs_and_extreme_scales(ora):
    """Truncation (not rounding) of the product, the sign of zero, the scale floor, overflow to
    infinity: whatever f32 gives, bit for bit."""
    k, n = 16, 16
    q = np.tile(np.array([0, 1, -1, 127, -127, -128, 3, -3, 64, -64, 5, 0, 100, -100, 2, -2], np.int8), (k, 1))
    s = np.array([1.0, -1.0, 1e-12, 3.0e38, 1.17549435e-38, 1e-45, 0.1, 1.0 / 3.0, 7.0e-3, 2.5,
                  0.0, -0.0, 1.0000001, 0.99999994, 123.456, 1e30], np.float32)
    want = ora.int8_to_bf16_per_channel(q, s)
    got = _run(q, s, k, n, 0)
    assert got.tobytes() == want.tobytes()
    assert got[0, 1] == 0xBF80 and got[0, 11] == 0x8000   # 1 * -1.0, 0 * -0.0 keeps the sign


def test_round_trip_error_bound(ora):
    """quantise -> dequantise on the device stays within half a step plus the bf16 truncation
    (the bound of the reference's own round-trip test, src/tensor/quantizer.rs:1050-1062)."""
    k, n, gs = 256, 512, 128
    w = _weights(9, k, n)
    q, s = capi.absmax_per_group_symmetric(w, gs)
    got = _run(q, s, k, n, gs)
    back = (got.astype(np.uint32) << 16).view(np.float32)
    step = np.repeat(s, gs, axis=0)[:k]
    assert (np.abs(back - w) <= 0.51 * step + np.abs(w) * 2.0 ** -7 + 1e-12).all()
    assert hip().hipDeviceSynchronize() == 0
