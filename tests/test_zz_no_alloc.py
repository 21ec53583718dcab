"""atenia_moe_hip_layer_forward_device_noalloc through the C ABI against
atenia_moe_hip_layer_forward_device: same kernels on another workspace (the library's static
buffer), so the outputs must be identical bit for bit -- on two calls in a row, the second with a
smaller batch, with another layer's call in between (the buffer keeps the last call's contents,
laid out for other dimensions), and for shapes whose h rows carry K padding that the call has to
zero itself.  The reference has no such entry point; the bar is the existing one's output, which
the other GPU tests hold against the CPU oracle."""
import numpy as np
import pytest

from ateniaengine_amd import capi
from tests import synth as S
from tests.hipmem import DeviceArray, Graph, Stream, mem_free

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _need_gpu():
    assert capi.available(), "no gfx950 device: the HIP path cannot run (there is no fallback)"


def _run(gL, x, noalloc, act=capi.ACT_F32, stream=0, watch_memory=False):
    T, d = x.shape
    if act == capi.ACT_BF16:
        dx = DeviceArray.from_host(capi.f32_to_bf16_trunc(x))
    else:
        dx = DeviceArray.from_host(x)
    out = DeviceArray((T, d), np.float32, fill=0xFF)
    fn = gL.forward_device_noalloc if noalloc else gL.forward_device
    before = mem_free() if watch_memory else 0
    fn(dx.ptr, act, T, out.ptr, stream)
    if watch_memory:  # the call must not have allocated (or freed) device memory
        after = mem_free()
        assert after == before, f"free device memory moved by {after - before} bytes across the call"
    assert gL.status(stream)[0] == 0
    return out.to_host()


CASES = [
    # name, E, k, d, f, f_s, gated, conv, wdtype
    ("bf16_padded_h", 12, 4, 128, 88, 352, True, 1, capi.WEIGHT_BF16),   # f, f_s % 32 != 0
    ("int8_padded_h", 5, 3, 72, 100, 36, True, 1, capi.WEIGHT_INT8_W8A16),
    ("bf16_plain", 8, 2, 256, 512, 0, False, 0, capi.WEIGHT_BF16),
    ("f32", 8, 2, 128, 256, 0, False, 0, capi.WEIGHT_F32),
    ("many_experts_bf16", 40, 2, 128, 96, 64, True, 1, capi.WEIGHT_BF16),  # logits scratch (E > 31)
    # per-group scales: streaming / mid-batch forms on the int8 blocks, the tiled kernels on the
    # layer's bf16 copy (made by the allocating call that runs first for each batch size)
    ("int8_per_group", 8, 2, 256, 512, 128, True, 1, capi.WEIGHT_INT8_PER_GROUP),
]


@pytest.mark.parametrize("name,E,k,d,f,f_s,gated,conv,wd", CASES)
def test_noalloc_equals_forward_device_twice_second_smaller(ora, name, E, k, d, f, f_s, gated,
                                                            conv, wd):
    W = S.make_weights(311, E, d, f, f_s=f_s, gated=gated)
    oL, gL = S.build_pair(ora, W, k, conv, wd)
    # a second layer of other dimensions scribbles over the static buffer between the calls
    W2 = S.make_weights(312, 6, 192, 160, f_s=96, gated=False)
    _, other = S.build_pair(ora, W2, 3, 0, capi.WEIGHT_BF16)
    bf16_rows = wd != capi.WEIGHT_F32
    with gL, other:
        # 300 takes the tiled kernels (split tail buffers) where they exist, 120 the mid-batch
        # kernel where the widths allow it, 37 that kernel for the down phase alone
        for T in (37, 9, 1, 120, 300):
            x = S.make_tokens(1000 + T, T, d, bf16=bf16_rows)
            want = _run(gL, x, noalloc=False)
            _run(gL, x, noalloc=True)  # warm: one-time kernel attributes, lazily made copies
            # whatever batch sizes were seen before, the call itself allocates nothing
            got = _run(gL, x, noalloc=True, watch_memory=True)
            assert got.tobytes() == want.tobytes(), f"{name} T={T}: no-alloc output differs"
            idx, w, counts, offsets, perm = gL.last_routing(T)  # taps read the static buffer
            o_idx, _ = oL.route_tokens(x)
            assert (idx == o_idx).all()
            oc, oo, op = ora.permute(o_idx, E)
            assert (counts == oc).all() and (offsets == oo).all() and (perm == op).all()
            _run(other, S.make_tokens(77, 21, 192), noalloc=True)
        if bf16_rows:  # bf16 activations: no bf16 copy of x is made, other workspace layout
            x = S.make_tokens(5, 24, d)
            assert (_run(gL, x, True, capi.ACT_BF16).tobytes()
                    == _run(gL, x, False, capi.ACT_BF16).tobytes())


def test_noalloc_rejects_what_does_not_fit(ora):
    W = S.make_weights(313, 8, 512, 1024)
    _, gL = S.build_pair(ora, W, 2, 0, capi.WEIGHT_BF16)
    with gL:
        T = 4096  # 8192 pairs x (2 * 1024 + 4 * 4 * 512) bytes: far beyond 16 MiB
        dx = DeviceArray((T, 512), np.float32, fill=0)
        out = DeviceArray((T, 512), np.float32, fill=0)
        with pytest.raises(capi.MoeHipError) as e:
            gL.forward_device_noalloc(dx.ptr, capi.ACT_F32, T, out.ptr)
        assert e.value.rc == capi.ERR_UNSUPPORTED and "static buffer" in str(e.value)
        # the handle is still usable, both ways
        x = S.make_tokens(3, 5, 512)
        assert _run(gL, x, True).tobytes() == _run(gL, x, False).tobytes()


@pytest.mark.parametrize("T", [8, 120, 300])
def test_noalloc_call_can_be_captured_and_replayed(ora, T):
    """The call only launches kernels (its workspace is initialised by a kernel, not a memset),
    so it can sit in a HIP graph: every replay, with eager work in between, equals the eager
    result for the input then in the buffer.  Batch sizes: the register-resident streaming
    kernels, the mid-batch kernel, the tiled kernels (with the split tail of their down launch)."""
    W = S.make_weights(314, 8, 256, 512)
    _, gL = S.build_pair(ora, W, 2, 0, capi.WEIGHT_BF16)
    with gL:
        d = 256
        want_family = {8: capi.KERNELS_STREAM, 120: capi.KERNELS_MID, 300: capi.KERNELS_TILED}[T]
        assert gL.expert_kernels(T)[0] == want_family
        s = Stream()
        dx = DeviceArray((T, d), np.float32, fill=0)
        out = DeviceArray((T, d), np.float32, fill=0)
        _run(gL, S.make_tokens(1, T, d), noalloc=True)  # warm: kernel attributes are set
        g = Graph(s)
        g.begin()
        gL.forward_device_noalloc(dx.ptr, capi.ACT_F32, T, out.ptr, s.ptr)
        g.end()
        from tests.hipmem import hip
        for rep in range(4):
            x = S.make_tokens(20 + rep, T, d)
            hip().hipMemcpy(dx.ptr, x.ctypes.data, x.nbytes, 1)
            g.launch()
            s.synchronize()
            got = out.to_host()
            want = _run(gL, x, noalloc=False)  # eager work between the replays
            assert got.tobytes() == want.tobytes(), f"replay {rep} differs"
        g.close()
        s.close()
