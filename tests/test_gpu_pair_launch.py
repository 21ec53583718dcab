"""Routed experts and a shared expert in ONE tiled launch per phase (bf16 pipelined kernels).

By default a bf16 layer with a shared expert runs the routed experts' and the shared expert's
tiles of a phase as one grid (gate/up: routed tiles first; down: the shared expert's first).  The
tiles are computed by the same code whichever launch carries them, so the outputs must be bit
for bit those of the separate launches -- on the handle's second stream (the arrangement that
ATENIA_MOE_PAIR_LAUNCHES=0 brings back; the library reads the knob once per process, so that run
is a child process) and one after the other on the caller's stream (the child with stage
profiling on).  The paired run itself is held against the oracle here.
"""
import hashlib
import os
import subprocess
import sys

import numpy as np
import pytest

from ateniaengine_amd import capi
from tests import synth as S
from tests.test_gpu_parity import TOL_BF16_TOY, check_layer

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

CASES = [
    # E, k, d, f, f_s, gated, T
    (8, 2, 256, 384, 256, True, 700),     # one row tile per expert, two for the shared expert
    (8, 2, 256, 384, 128, True, 1500),    # tiles of nine groups, split tail in the down launch
    (4, 2, 128, 256, 1024, False, 1100),  # shared expert four times as wide: the longer K first
    (16, 4, 256, 128, 512, True, 2100),   # many short tiles next to a wide shared expert
]


def _outputs(ora, case, profiling):
    E, k, d, f, fs, gated, T = case
    W = S.make_weights(7300 + T, E, d, f, f_s=fs, gated=gated, router_std=0.05 / np.sqrt(d))
    outs = []
    _, gL = S.build_pair(ora, W, k, capi.CONVENTION_HUGGINGFACE_QWEN, capi.WEIGHT_BF16)
    with gL:
        plan = gL.plan(T)
        assert plan["up"] == plan["down"] == capi.KERNELS_TILED, plan
        assert plan["shared_up"] == plan["shared_down"] == capi.KERNELS_TILED, plan
        gL.set_profiling(profiling)
        for i in range(3):
            outs.append(gL.forward(S.make_tokens(7400 + T + i, T, d)).copy())
        outs.append(gL.forward(S.make_tokens(7400 + T, T, d)).copy())  # the first one again
    assert outs[3].tobytes() == outs[0].tobytes()
    return [hashlib.sha256(o.tobytes()).hexdigest() for o in outs[:3]]


CHILD = r"""
from oracle import moe_oracle as ora
from tests.test_gpu_pair_launch import CASES, _outputs
ora.build()
for i, case in enumerate(CASES):
    for prof in (False, True):
        print("sha", i, int(prof), " ".join(_outputs(ora, case, prof)), flush=True)
print("child ok")
"""


@pytest.fixture(scope="module")
def separate_launches():
    env = dict(os.environ, ATENIA_MOE_PAIR_LAUNCHES="0", PYTHONPATH=ROOT)
    r = subprocess.run([sys.executable, "-u", "-c", CHILD], cwd=ROOT, env=env, capture_output=True,
                       text=True, timeout=900)
    assert r.returncode == 0 and "child ok" in r.stdout, (r.stdout[-3000:], r.stderr[-3000:])
    got = {}
    for ln in r.stdout.splitlines():
        if ln.startswith("sha "):
            _, i, prof, *h = ln.split()
            got[(int(i), int(prof))] = h
    return got


@pytest.mark.parametrize("i", range(len(CASES)))
def test_paired_launch_equals_separate_launches(ora, separate_launches, i):
    case = CASES[i]
    E, k, d, f, fs, gated, T = case
    assert capi.available(), "no gfx950 device: the HIP path cannot run (there is no fallback)"
    W = S.make_weights(7300 + T, E, d, f, f_s=fs, gated=gated, router_std=0.05 / np.sqrt(d))
    oL, gL = S.build_pair(ora, W, k, capi.CONVENTION_HUGGINGFACE_QWEN, capi.WEIGHT_BF16)
    with gL:
        check_layer(ora, oL, gL, S.make_tokens(7400 + T, T, d), TOL_BF16_TOY, sample=range(0, T, 31))
    mine = _outputs(ora, case, False)
    assert mine == _outputs(ora, case, True), "stage profiling changed the result"
    assert mine == separate_launches[(i, 0)], "differs from the launches on the second stream"
    assert mine == separate_launches[(i, 1)], "differs from the two launches on one stream"
