"""Runs the C++ tests of the weight-ingestion side of the host mirror
(tests/host/moe_ingest_test.cpp).  The binary reads the golden layer files itself; this wrapper
only writes a small safetensors file that holds one [4, 6] tensor three times (F32, BF16, F16,
values exact in all three, subnormals and infinities included) and the f32 bits they must
widen to."""
import json
import os
import struct
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "host", "moe_ingest_test")
GOLDEN = os.path.join(ROOT, "tests", "golden")


def _write_dtype_file(work):
    # exact in f16 (hence in bf16 only when <= 8 significant bits: keep 3-bit mantissas)
    vals = np.array([0.0, -0.0, 1.0, -1.0, 0.5, 1.5, -2.75 + 0.25, 3.0, 6.0, -12.0, 0.125, 1024.0,
                     2.0 ** -14, -(2.0 ** -14), 2.0 ** -20, -(2.0 ** -24), 1.25 * 2.0 ** -16, 65504.0 - 65504.0 + 57344.0,
                     np.inf, -np.inf, 1.75, -0.875, 40.0, -448.0], dtype=np.float32).reshape(4, 6)
    f16 = vals.astype(np.float16)
    assert np.array_equal(f16.astype(np.float32), vals, equal_nan=True)
    bf16 = (vals.view(np.uint32) >> 16).astype(np.uint16)
    assert np.array_equal((bf16.astype(np.uint32) << 16).view(np.float32), vals)
    parts = [("t.f32", "F32", vals.tobytes()), ("t.bf16", "BF16", bf16.tobytes()), ("t.f16", "F16", f16.tobytes()),
             ("t.i64", "I64", np.arange(24, dtype=np.int64).tobytes())]
    header, blob = {"__metadata__": {"format": "pt"}}, b""
    for name, dtype, raw in parts:
        header[name] = {"dtype": dtype, "shape": [4, 6], "data_offsets": [len(blob), len(blob) + len(raw)]}
        blob += raw
    text = json.dumps(header).encode()
    text += b" " * (-len(text) % 8)
    with open(os.path.join(work, "dtypes.safetensors"), "wb") as fp:
        fp.write(struct.pack("<Q", len(text)) + text + blob)
    vals.tofile(os.path.join(work, "dtypes_expected.bin"))


def _run(work, extra):
    if not os.path.exists(BIN):
        pytest.fail("tests/host/moe_ingest_test is not built (run __graft_entry__.build())")
    _write_dtype_file(work)
    r = subprocess.run([BIN, GOLDEN, work] + extra, capture_output=True, text=True, timeout=300)
    print(r.stdout)
    print(r.stderr)
    return r


def test_ingest_logic_without_gpu(tmp_path):
    """Names, weight map, classic and packed binding, error texts, the safetensors reader, and
    the golden layer files assembled and checked through the CPU oracle."""
    from ateniaengine_amd import capi

    if capi.available():
        pytest.skip("a GPU is present: covered by the device run below")
    r = _run(str(tmp_path), ["--no-gpu"])
    assert r.returncode == 0, r.stdout
    assert "golden_layers_through_the_oracle_match_f64_refs" in r.stdout and " 0 failed" in r.stdout


@pytest.mark.gpu
def test_ingest_to_forward_on_device(tmp_path):
    r = _run(str(tmp_path), [])
    assert r.returncode == 0, r.stdout + r.stderr
    assert "atenia_mode_matches_atenia_ref" in r.stdout and " 0 failed" in r.stdout
