"""Threading contract of the boundary: any host thread may call; different handles run
concurrently (each on its own stream); calls on ONE handle are serialised by the handle's mutex
(the reference serialises every MoE forward behind its registry lock, src/moe/graph_op.rs:221-224,
304-316).  ctypes drops the GIL for the duration of a call, so these threads really overlap.
Every concurrent result must equal the single-threaded one bit for bit."""
import threading

import numpy as np
import pytest

from ateniaengine_amd import capi
from tests import synth as S
from tests.hipmem import DeviceArray, Stream

pytestmark = pytest.mark.gpu

# (weight dtype, E, k, d, f, shared f, tokens)
SHAPES = [
    (capi.WEIGHT_BF16, 8, 2, 256, 512, 0, 1),
    (capi.WEIGHT_INT8_W8A16, 8, 2, 256, 512, 0, 7),
    (capi.WEIGHT_BF16, 60, 4, 128, 192, 256, 130),    # > 32 router rows, shared expert, tiled kernels
    (capi.WEIGHT_F32, 4, 2, 64, 96, 0, 9),
]


def _run_threads(workers):
    errors = []

    def guard(fn):
        def run():
            try:
                fn()
            except BaseException as e:  # noqa: BLE001 - reported by the main thread
                errors.append(e)
        return run

    ts = [threading.Thread(target=guard(w)) for w in workers]
    for t in ts:
        t.start()
    for t in ts:
        t.join(timeout=100)
    assert not any(t.is_alive() for t in ts), "a worker thread did not finish"
    if errors:
        raise errors[0]


def test_handles_run_concurrently_from_their_own_threads(ora):
    layers, inputs, want = [], [], []
    for i, (wd, E, k, d, f, fs, T) in enumerate(SHAPES):
        W = S.make_weights(700 + i, E, d, f, f_s=fs, gated=fs > 0, router_std=1.0 / np.sqrt(d))
        conv = capi.CONVENTION_HUGGINGFACE_QWEN if fs else capi.CONVENTION_ATENIA
        _, gL = S.build_pair(ora, W, k, conv, wd, max_tokens_hint=T)
        xs = [S.make_tokens(900 + 10 * i + j, T, d) for j in range(3)]
        layers.append(gL)
        inputs.append(xs)
        want.append([gL.forward(x).copy() for x in xs])   # single-threaded results
    rounds = 12
    got = [[None] * rounds for _ in layers]

    def host_worker(i):
        def run():
            for r in range(rounds):
                got[i][r] = layers[i].forward(inputs[i][r % 3]).copy()
        return run

    try:
        _run_threads([host_worker(i) for i in range(len(layers))])
        for i in range(len(layers)):
            for r in range(rounds):
                assert got[i][r].tobytes() == want[i][r % 3].tobytes(), f"layer {i}, round {r}"

        # the device entry point on caller-owned streams, one stream per thread
        def device_worker(i):
            def run():
                T, d = inputs[i][0].shape
                stream = Stream()
                dx = [DeviceArray.from_host(x) for x in inputs[i]]
                dout = DeviceArray((T, d), np.float32, fill=0)
                for r in range(rounds):
                    layers[i].forward_device(dx[r % 3].ptr, capi.ACT_F32, T, dout.ptr, stream.ptr)
                    stream.synchronize()
                    got[i][r] = dout.to_host().copy()
                stream.close()
            return run

        _run_threads([device_worker(i) for i in range(len(layers))])
        for i in range(len(layers)):
            for r in range(rounds):
                assert got[i][r].reshape(-1).tobytes() == want[i][r % 3].reshape(-1).tobytes(), \
                    f"device entry, layer {i}, round {r}"
    finally:
        for gL in layers:
            gL.close()


def test_one_handle_shared_by_threads_is_serialised(ora):
    wd, E, k, d, f, fs, T = SHAPES[2]
    W = S.make_weights(777, E, d, f, f_s=fs, gated=True, router_std=1.0 / np.sqrt(d))
    _, gL = S.build_pair(ora, W, k, capi.CONVENTION_HUGGINGFACE_QWEN, wd)
    # different batch sizes per thread, so the shared workspace is re-sized and re-used across
    # callers; an unserialised call would read another call's grouping
    sizes = [1, 5, 40, T]
    xs = [S.make_tokens(40 + n, n, d) for n in sizes]
    with gL:
        want = [gL.forward(x).copy() for x in xs]
        rounds = 10
        got = [[None] * rounds for _ in sizes]

        def worker(i):
            def run():
                for r in range(rounds):
                    got[i][r] = gL.forward(xs[i]).copy()
            return run

        _run_threads([worker(i) for i in range(len(sizes))])
        for i in range(len(sizes)):
            for r in range(rounds):
                assert got[i][r].tobytes() == want[i].tobytes(), f"{sizes[i]} tokens, round {r}"


def test_one_handle_on_two_streams_is_ordered_on_the_device(ora):
    """The asynchronous entry point on ONE handle from two streams, calls issued back to back
    without any host synchronisation in between: the second stream must wait for the first
    stream's kernels (they share the handle's workspace), so every output equals the result of the
    same call made alone."""
    wd, E, k, d, f, fs, _ = SHAPES[2]
    W = S.make_weights(778, E, d, f, f_s=fs, gated=True, router_std=1.0 / np.sqrt(d))
    _, gL = S.build_pair(ora, W, k, capi.CONVENTION_HUGGINGFACE_QWEN, wd, max_tokens_hint=700)
    sizes = [700, 3, 260, 1, 64, 700]  # long and short calls alternate between the streams
    xs = [S.make_tokens(60 + i, n, d) for i, n in enumerate(sizes)]
    with gL:
        want = [gL.forward(x).copy() for x in xs]
        streams = [Stream(), Stream()]
        dx = [DeviceArray.from_host(x) for x in xs]
        for rep in range(3):
            outs = [DeviceArray(x.shape, np.float32, fill=0) for x in xs]
            for i, n in enumerate(sizes):
                gL.forward_device(dx[i].ptr, capi.ACT_F32, n, outs[i].ptr, streams[i % 2].ptr)
            for s in streams:
                s.synchronize()
            for i in range(len(sizes)):
                assert outs[i].to_host().tobytes() == want[i].tobytes(), \
                    f"repeat {rep}, call {i} ({sizes[i]} tokens)"
        for s in streams:
            s.close()
