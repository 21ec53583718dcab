"""Runs the C++ tests of the host mirror (tests/host/host_mirror_test.cpp).  The golden layer
fixtures are handed to the binary as one flat file: per layer a 32-byte name, six int32
(E, k, d, f, f_shared, gated) and the f32 arrays router, gate, up, down, shared gate/up/down,
shared-expert gate vector, input, atenia_ref, hf_ref."""
import os
import struct
import subprocess

import numpy as np
import pytest

from tests import golden_io as G

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "host", "host_mirror_test")


def _write_fixtures(path, names):
    with open(path, "wb") as fp:
        fp.write(struct.pack("<i", len(names)))
        for name in names:
            A = G.layer_arrays(name)
            side = G.sidecar(name)
            E, f, d = A["w_gate"].shape
            fs = A["s_gate"].shape[0] if A.get("s_gate") is not None else 0
            gated = A.get("shared_gate") is not None
            fp.write(name.encode().ljust(32, b"\0"))
            fp.write(struct.pack("<6i", E, int(side["experts_per_token"]), d, f, fs, int(gated)))
            order = ["w_router", "w_gate", "w_up", "w_down"]
            if fs:
                order += ["s_gate", "s_up", "s_down"]
            if gated:
                order += ["shared_gate"]
            for key in order:
                fp.write(np.ascontiguousarray(A[key], dtype=np.float32).tobytes())
            for key in ("input", "atenia_ref", "hf_ref"):
                fp.write(np.asarray(side[key], dtype=np.float32).tobytes())


def _run(args):
    if not os.path.exists(BIN):
        pytest.fail("tests/host/host_mirror_test is not built (run __graft_entry__.build())")
    r = subprocess.run([BIN] + args, capture_output=True, text=True, timeout=300)
    print(r.stdout)
    print(r.stderr)
    return r


def test_host_logic_without_gpu(tmp_path):
    """Config validation, registry, error texts, and the loud failure of a forward when no
    device is present (this container has none)."""
    from ateniaengine_amd import capi

    if capi.available():
        pytest.skip("a GPU is present: covered by the device run below")
    r = _run([os.devnull, "--no-gpu"])
    assert r.returncode == 0, r.stdout
    assert "forward_without_device_fails_loudly" in r.stdout


@pytest.mark.gpu
def test_host_mirror_on_device(tmp_path):
    path = str(tmp_path / "fixtures.bin")
    _write_fixtures(path, ["mixtral_layer0", "qwen15_moe_layer0"])
    r = _run([path])
    assert r.returncode == 0, r.stdout + r.stderr
    assert " 0 failed" in r.stdout
