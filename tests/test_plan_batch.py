"""Which expert kernels a batch takes (`atenia_moe_hip_plan_batch`: a pure function of the layer's
dimensions and the batch size, no device needed).

The reference has one expert loop for every batch size (src/moe/layer.rs:405-443), so there is
nothing to compare the choice with; what can be held is that the plan is *defensible*: defined for
every shape, ordered in T (register-resident streaming -> mid-batch -> matrix-core tiled, never
back, per phase), and consistent with what the kernels can take.  Shapes: every layer the random
GPU suites draw (tests/test_gpu_fuzz.py), the five benchmark configurations, and two shapes of
the reference's model families (src/moe/family.rs) outside the benchmark list: Mixtral-8x22B
(d = 6144, f = 16384) and a 128-expert top-8 layer with narrow experts (f = 768).
"""
import numpy as np
import pytest

from ateniaengine_amd import capi
from tests.test_gpu_fuzz import _cases, _mid_cases

FAMILY_ORDER = {capi.KERNELS_STREAM: 0, capi.KERNELS_MID: 1, capi.KERNELS_TILED: 2}

NAMED = [
    # E, k, d, f, f_s, weight dtype
    (8, 2, 1024, 2048, 0, capi.WEIGHT_F32),              # config 1
    (8, 2, 4096, 14336, 0, capi.WEIGHT_BF16),            # config 2
    (8, 2, 4096, 14336, 0, capi.WEIGHT_INT8_W8A16),      # config 3
    (8, 2, 4096, 14336, 0, capi.WEIGHT_INT8_PER_GROUP),
    (60, 4, 2048, 1408, 5632, capi.WEIGHT_BF16),         # config 4
    (64, 6, 2048, 1408, 2816, capi.WEIGHT_BF16),         # config 5
    (8, 2, 6144, 16384, 0, capi.WEIGHT_BF16),            # Mixtral-8x22B
    (8, 2, 6144, 16384, 0, capi.WEIGHT_INT8_W8A16),
    (128, 8, 2048, 768, 0, capi.WEIGHT_BF16),            # many narrow experts
    (128, 8, 2048, 768, 768, capi.WEIGHT_BF16),
    (256, 8, 7168, 2048, 2048, capi.WEIGHT_BF16),        # DeepSeek-V3 routed-expert shape
]


def _shapes():
    seen = []
    for p in _cases(150, 20240607) + _mid_cases(60, 20250311):
        E, k, d, f, fs, _g, _c, wd, _T, _s = p.values
        seen.append((E, k, d, f, fs, wd))
    return sorted(set(seen)) + NAMED


def _batch_sizes():
    ts = set(range(1, 701)) | {int(round(v)) for v in np.geomspace(700, 40000, 160)}
    return sorted(ts)


@pytest.mark.parametrize("E,k,d,f,fs,wd", _shapes())
def test_plan_is_defined_and_ordered_in_the_batch_size(E, k, d, f, fs, wd):
    gs = 128 if wd == capi.WEIGHT_INT8_PER_GROUP else 0
    prev = None
    for T in _batch_sizes():
        p = capi.plan_batch(E, k, d, f, fs, wd, T, group_size=gs)
        if wd == capi.WEIGHT_F32:
            assert p["up"] == p["down"] == capi.KERNELS_F32
            assert p["shared_up"] == p["shared_down"] == (capi.KERNELS_F32 if fs else -1)
            assert not (p["y_bf16"] or p["ys_bf16"] or p["tall_tiles"] or p["duo"])
            continue
        assert p["up"] in FAMILY_ORDER and p["down"] in FAMILY_ORDER, (T, p)
        assert (p["shared_up"] == -1) == (fs == 0) and (p["shared_down"] == -1) == (fs == 0), (T, p)
        # bf16 expert outputs: only bf16 layers, only behind the matrix-core down launch
        if p["y_bf16"]:
            assert wd == capi.WEIGHT_BF16 and p["down"] == capi.KERNELS_TILED, (T, p)
        if p["ys_bf16"]:
            assert p["y_bf16"] and p["shared_down"] == capi.KERNELS_TILED, (T, p)
        if p["tall_tiles"]:
            assert capi.KERNELS_TILED in (p["up"], p["down"]), (T, p)
            # a W8A16 layer has them on the bf16 copy of its int8 values only
            assert wd != capi.WEIGHT_INT8_W8A16 or p["int8_copy"], (T, p)
        if p["int8_copy"]:
            assert wd == capi.WEIGHT_INT8_W8A16 and p["up"] == p["down"] == capi.KERNELS_TILED, (T, p)
            assert fs == 0 or p["shared_up"] == p["shared_down"] == capi.KERNELS_TILED, (T, p)
            assert not p["y_bf16"], (T, p)
        if prev is not None and prev[1]["int8_copy"]:
            assert p["int8_copy"], f"back from the bf16 copy at T={T}"
        assert p["duo"] == 0, "the two-workgroup form is off unless ATENIA_MOE_DUO_MAX_K asks for it"
        if prev is not None:
            for phase in ("up", "down"):
                assert FAMILY_ORDER[p[phase]] >= FAMILY_ORDER[prev[1][phase]], (
                    f"{phase} phase goes back from {prev[1][phase]} at T={prev[0]} to {p[phase]} at T={T}")
        prev = (T, p)
    # a large enough batch ends on the matrix cores wherever the widths allow it (K in whole 64-k
    # stages; other widths keep the streaming kernels, which take any K)
    if wd != capi.WEIGHT_F32 and d % 64 == 0 and f % 64 == 0:
        assert prev[1]["up"] == prev[1]["down"] == capi.KERNELS_TILED, prev


def test_plan_rejects_what_create_rejects():
    for bad in [dict(E=0), dict(k=0), dict(k=9), dict(d=0), dict(f=0), dict(fs=-1), dict(wd=7), dict(T=0)]:
        a = dict(E=8, k=2, d=256, f=512, fs=0, wd=capi.WEIGHT_BF16, T=16)
        a.update(bad)
        with pytest.raises(capi.MoeHipError):
            capi.plan_batch(a["E"], a["k"], a["d"], a["f"], a["fs"], a["wd"], a["T"])
    with pytest.raises(capi.MoeHipError):  # per-group scales need a group size in whole 64-k blocks
        capi.plan_batch(8, 2, 256, 512, 0, capi.WEIGHT_INT8_PER_GROUP, 16, group_size=100)
