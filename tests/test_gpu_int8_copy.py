"""W8A16 layers on the bf16 tiled kernels: from 256 rows per expert on average the tiled phases
run on a bf16 copy of the layer's int8 values (exact: every int8 is a bf16 value) and the row
scales multiply the f32 results, instead of the int8 tiled kernel that widens the weights next to
its matrix instructions.  Same products, same k order: the outputs must stay within the bars of
every other kernel against the oracle, and within f32 rounding noise of the int8 kernel's, which
ATENIA_MOE_INT8_COPY_MIN_ROWS=0 brings back (the library reads the knob once per process, so
that run is a child process).
"""
import hashlib
import os
import subprocess
import sys

import numpy as np
import pytest

from ateniaengine_amd import capi
from tests import synth as S
from tests.hipmem import DeviceArray
from tests.test_gpu_parity import TOL_BF16_TOY, check_layer

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

CASES = [
    # E, k, d, f, f_s, gated, T, on the copy
    (8, 2, 256, 384, 0, False, 1100, True),      # 275 rows: tiles of nine groups, split tail
    (4, 2, 128, 256, 128, True, 700, True),      # shared expert (second stream), gated
    (8, 2, 256, 512, 256, False, 1500, True),    # shared expert, ungated; 375 rows
    (3, 2, 192, 320, 0, False, 1025, True),      # column tiles past N in both phases
    (8, 2, 256, 384, 0, False, 900, False),      # 225 rows: the int8 tiled kernel keeps it
    (8, 2, 200, 392, 0, False, 1300, True),      # K padded to whole 64-k stages in both phases
    (8, 2, 64, 192, 0, False, 1300, False),      # K of the gate/up phase below two stages: no copy
]


def _layer(ora, case):
    E, k, d, f, fs, gated, T, _ = case
    W = S.make_weights(8100 + T, E, d, f, f_s=fs, gated=gated, router_std=0.05 / np.sqrt(d),
                       outlier_frac=0.02)
    conv = capi.CONVENTION_HUGGINGFACE_QWEN if fs else capi.CONVENTION_ATENIA
    return S.build_pair(ora, W, k, conv, capi.WEIGHT_INT8_W8A16)


def _outputs(ora, case):
    T, d = case[6], case[2]
    oL, gL = _layer(ora, case)
    with gL:
        outs = [gL.forward(S.make_tokens(8200 + T + i, T, d)).copy() for i in range(2)]
    return outs


CHILD = r"""
import numpy as np
from oracle import moe_oracle as ora
from tests.test_gpu_int8_copy import CASES, _outputs
ora.build()
for i, case in enumerate(CASES):
    for j, o in enumerate(_outputs(ora, case)):
        np.save(f"{OUT}/i8_{i}_{j}.npy", o)
print("child ok")
"""


@pytest.fixture(scope="module")
def int8_kernel_outputs(tmp_path_factory):
    out = tmp_path_factory.mktemp("int8_kernel")
    env = dict(os.environ, ATENIA_MOE_INT8_COPY_MIN_ROWS="0", PYTHONPATH=ROOT)
    r = subprocess.run([sys.executable, "-u", "-c", f"OUT = {str(out)!r}\n" + CHILD], cwd=ROOT,
                       env=env, capture_output=True, text=True, timeout=900)
    assert r.returncode == 0 and "child ok" in r.stdout, (r.stdout[-3000:], r.stderr[-3000:])
    return out


@pytest.mark.parametrize("i", range(len(CASES)))
def test_bf16_copy_of_the_int8_values(ora, int8_kernel_outputs, i):
    case = CASES[i]
    E, k, d, f, fs, gated, T, on_copy = case
    oL, gL = _layer(ora, case)
    with gL:
        plan = gL.plan(T)
        assert plan["up"] == plan["down"] == capi.KERNELS_TILED, plan
        assert plan["int8_copy"] == int(on_copy) and plan["tall_tiles"] == int(on_copy), plan
        assert not plan["y_bf16"], plan
        x = S.make_tokens(8200 + T, T, d)
        check_layer(ora, oL, gL, x, TOL_BF16_TOY, sample=range(0, T, 29))
        # smaller batches afterwards go back to the int8 blocks, larger ones to the copy again
        for T2 in (16, 300, T):
            x2 = S.make_tokens(8300 + T2, T2, d)
            check_layer(ora, oL, gL, x2, TOL_BF16_TOY, sample=range(0, T2, max(1, T2 // 24)))
    mine = _outputs(ora, case)
    for j, o in enumerate(mine):
        other = np.load(int8_kernel_outputs / f"i8_{i}_{j}.npy")
        bar = 2e-5 * float(np.abs(other).max())
        assert float(np.abs(o - other).max()) <= bar, "differs from the int8 tiled kernel's result"


def test_noalloc_entry_needs_the_copy_to_exist(ora):
    """The entry point that allocates nothing cannot make the copy: it says so until an allocating
    call (or max_tokens_hint at create) has made it, and runs on it afterwards."""
    case = CASES[0]
    E, k, d, f, fs, gated, T, _ = case
    oL, gL = _layer(ora, case)
    x = S.make_tokens(8400, T, d)
    with gL:
        dx = DeviceArray.from_host(x)
        a = DeviceArray((T, d), np.float32, fill=0)
        b = DeviceArray((T, d), np.float32, fill=0)
        with pytest.raises(capi.MoeHipError, match="bf16 copy"):
            gL.forward_device_noalloc(dx.ptr, capi.ACT_F32, T, a.ptr)
        gL.forward_device(dx.ptr, capi.ACT_F32, T, a.ptr)
        gL.forward_device_noalloc(dx.ptr, capi.ACT_F32, T, b.ptr)
        assert gL.status()[0] == 0
        ha, hb = a.to_host(), b.to_host()
        assert hashlib.sha256(ha.tobytes()).hexdigest() == hashlib.sha256(hb.tobytes()).hexdigest()


CAPPED = r"""
import numpy as np
from ateniaengine_amd import capi
from oracle import moe_oracle as ora
from tests import synth as S
from tests.test_gpu_int8_copy import CASES, _layer
from tests.test_gpu_parity import TOL_BF16_TOY, check_layer
ora.build()
for case in (CASES[0], CASES[2]):
    E, k, d, f, fs, gated, T, _ = case
    oL, gL = _layer(ora, case)
    with gL:
        assert gL.plan(T)["int8_copy"] == 1  # what the dimensions alone say
        x = S.make_tokens(8500 + T, T, d)
        out, _ = check_layer(ora, oL, gL, x, TOL_BF16_TOY, sample=range(0, T, 37))
        assert gL.expert_kernels(T)[0] == capi.KERNELS_TILED
        np.save(f"{OUT}/capped_{T}.npy", out)
        check_layer(ora, oL, gL, S.make_tokens(8600, 40, d), TOL_BF16_TOY)
        out2, _ = check_layer(ora, oL, gL, x, TOL_BF16_TOY, sample=range(0, T, 37))
        assert out2.tobytes() == out.tobytes()
print("child ok")
"""


def test_layer_keeps_the_int8_kernels_when_the_copy_cannot_be_made(ora, tmp_path):
    """The copy is an optimisation: when it cannot be made (here: a cap of 0 MiB on its size, the
    same path an allocation failure takes) the forward still runs, on the int8 tiled kernels, with
    their results -- in that call and in every later one."""
    env = dict(os.environ, ATENIA_MOE_INT8_COPY_MAX_MB="0", PYTHONPATH=ROOT)
    r = subprocess.run([sys.executable, "-u", "-c", f"OUT = {str(tmp_path)!r}\n" + CAPPED], cwd=ROOT,
                       env=env, capture_output=True, text=True, timeout=900)
    assert r.returncode == 0 and "child ok" in r.stdout, (r.stdout[-3000:], r.stderr[-3000:])
    env0 = dict(os.environ, ATENIA_MOE_INT8_COPY_MIN_ROWS="0", PYTHONPATH=ROOT)
    r0 = subprocess.run([sys.executable, "-u", "-c",
                         f"OUT = {str(tmp_path)!r}\n" + CAPPED.replace("capped_", "int8_").replace(
                             'assert gL.plan(T)["int8_copy"] == 1', 'assert gL.plan(T)["int8_copy"] == 0')],
                        cwd=ROOT, env=env0, capture_output=True, text=True, timeout=900)
    assert r0.returncode == 0 and "child ok" in r0.stdout, (r0.stdout[-3000:], r0.stderr[-3000:])
    for case in (CASES[0], CASES[2]):
        T = case[6]
        a, b = np.load(tmp_path / f"capped_{T}.npy"), np.load(tmp_path / f"int8_{T}.npy")
        assert a.tobytes() == b.tobytes(), "not the int8 tiled kernels' result"
