"""A warm handle's device entry points launch kernels only (no allocation, no memset, no
synchronisation), so a serving loop can capture a forward into a HIP graph and replay it.  Every
replay -- with new activations in the same buffers and eager work in between -- must give the
eager result bit for bit."""
import numpy as np
import pytest

from ateniaengine_amd import capi
from tests import synth as S
from tests.hipmem import DeviceArray, Graph, Stream, hip

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("wd,T,k,shared", [(capi.WEIGHT_BF16, 1, 2, False), (capi.WEIGHT_BF16, 8, 3, True),
                                           (capi.WEIGHT_INT8_W8A16, 1, 2, False), (capi.WEIGHT_BF16, 300, 2, False),
                                           (capi.WEIGHT_BF16, 100, 2, True), (capi.WEIGHT_INT8_W8A16, 150, 2, False),
                                           # tiled kernels with a shared expert: a bf16 layer carries its
                                           # tiles in the routed experts' launches; an int8 layer's eager calls
                                           # put its launches on the handle's second stream, a captured one
                                           # must not
                                           (capi.WEIGHT_BF16, 700, 2, True), (capi.WEIGHT_INT8_W8A16, 700, 2, True)])
def test_forward_replays_from_a_graph(ora, wd, T, k, shared):
    d = 256
    W = S.make_weights(40 + T, 8, d, 512, f_s=128 if shared else 0, gated=shared, router_std=1.0 / 16.0)
    conv = capi.CONVENTION_HUGGINGFACE_QWEN if shared else capi.CONVENTION_ATENIA
    _, gL = S.build_pair(ora, W, k, conv, wd, max_tokens_hint=T)
    xs = [S.make_tokens(100 + i, T, d) for i in range(4)]
    with gL:
        stream = Stream()
        dx = DeviceArray.from_host(xs[0])
        dout = DeviceArray((T, d), np.float32, fill=0)
        gL.forward_device(dx.ptr, capi.ACT_F32, T, dout.ptr, stream.ptr)  # warm: sizes every buffer
        stream.synchronize()
        g = Graph(stream)
        g.begin()
        gL.forward_device(dx.ptr, capi.ACT_F32, T, dout.ptr, stream.ptr)
        g.end()
        for i, x in enumerate(xs):
            want = gL.forward(x).reshape(T, d)        # eager, host buffers, the handle's own stream
            rc = hip().hipMemcpy(dx.ptr, np.ascontiguousarray(x).ctypes.data, x.nbytes, 1)
            assert rc == 0
            g.launch()
            stream.synchronize()
            assert dout.to_host().tobytes() == want.tobytes(), f"replay {i} differs from the eager forward"
        g.close()
        stream.close()
