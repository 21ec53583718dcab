"""The tiled kernel form with two workgroups per compute unit (csrc/ffn_tiled_duo.hip).

It is off by default (on MI355X it measured no faster than the 256-row form: its loop is bound by
LDS bandwidth) and is switched on by ATENIA_MOE_DUO_MAX_K, which the library reads once per
process.  So the cases below run in ONE child process with the knob set: same bars as the fixed
cases of test_gpu_parity.py (routing and grouping bit-exact, outputs within tolerance of the f64
reference and within 1e-3 of the arithmetic model), on shapes that exercise 128-row halves with
and without rows, column tiles past N, a shared expert beside the routed ones, and the bf16
expert outputs of its down phase.
"""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

CHILD = r"""
import numpy as np
from ateniaengine_amd import capi
from oracle import moe_oracle as ora
from tests import synth as S
from tests.test_gpu_parity import TOL_BF16_TOY, check_layer

ora.build()
assert capi.available()
cases = [
    # E, k, d, f, f_s, gated, conv, T
    (8, 2, 256, 512, 0, False, 0, 700),     # 175 rows per expert: a full half and a partial one
    (8, 2, 256, 512, 0, False, 0, 1100),    # two row tiles for some experts
    (4, 2, 128, 192, 64, True, 1, 600),     # column tiles past N in both phases, gated shared expert
    (17, 3, 320, 448, 128, False, 1, 900),  # 20 down strips, skew from 17 experts
    (60, 4, 256, 128, 0, False, 1, 2000),   # many experts, short K in the down phase
]
for i, (E, k, d, f, fs, gated, conv, T) in enumerate(cases):
    W = S.make_weights(5100 + i, E, d, f, f_s=fs, gated=gated, router_std=1.0 / np.sqrt(d))
    oL, gL = S.build_pair(ora, W, k, conv, capi.WEIGHT_BF16)
    with gL:
        plan = gL.plan(T)
        assert plan["up"] == plan["down"] == capi.KERNELS_TILED and plan["duo"] == 3, plan
        assert plan["y_bf16"] == 1 and plan["tall_tiles"] == 0, plan
        x = S.make_tokens(5200 + i, T, d)
        sample = sorted(set(np.linspace(0, T - 1, 64).astype(int).tolist()))
        _, worst = check_layer(ora, oL, gL, x, TOL_BF16_TOY, sample=sample)
        print(f"case {i}: E={E} k={k} d={d} f={f} f_s={fs} T={T}: max rel err {worst:.2e}", flush=True)
print("duo ok")
"""


def test_two_workgroup_form_in_a_process_that_switches_it_on():
    env = dict(os.environ, ATENIA_MOE_DUO_MAX_K="2048", PYTHONPATH=ROOT)
    r = subprocess.run([sys.executable, "-u", "-c", CHILD], cwd=ROOT, env=env, capture_output=True,
                       text=True, timeout=900)
    assert r.returncode == 0 and "duo ok" in r.stdout, (r.stdout[-3000:], r.stderr[-3000:])
