"""Per-group (Q8_0-style) int8: the oracle's restatement of absmax_per_group_symmetric
(src/tensor/quantizer.rs:175-248) pinned by closed forms, the library's row-major quantiser held
against it, and the GPU layer run on per-group weights against the oracle layer run on the
dequantised weights (q * scale, what the reference's CPU path computes with)."""
import numpy as np
import pytest

from ateniaengine_amd import capi
from tests import synth as S


# ---- the oracle's quantiser: closed forms ----------------------------------------------------
def test_group_maximum_maps_to_127_and_outlier_stays_local(ora):
    k, n, gs = 256, 3, 128
    w = np.full((k, n), 0.5, dtype=np.float32)
    w[5, 1] = -4.0     # an outlier in group 0 of column 1
    w[200, 2] = 1.0    # the maximum of group 1 of column 2
    q, s = ora.absmax_per_group_symmetric(w, gs)
    assert s.shape == (2, n)
    assert s[0, 1] == np.float32(4.0) / np.float32(127.0) and q[5, 1] == -127
    assert q[6, 1] == round(0.5 / float(s[0, 1]))          # coarse next to the outlier ...
    assert s[1, 1] == np.float32(0.5) / np.float32(127.0) and q[130, 1] == 127   # ... fine elsewhere
    assert q[200, 2] == 127 and q[201, 2] == 64            # 0.5 / (1/127) = 63.5 -> away from zero
    assert (q[:, 0] == 127).all()


def test_zero_group_gets_the_floor_and_partial_last_group(ora):
    k, n, gs = 200, 2, 128                                  # second group holds 72 rows
    w = np.zeros((k, n), dtype=np.float32)
    w[150, 1] = 2.0
    q, s = ora.absmax_per_group_symmetric(w, gs)
    assert s.shape == (2, n) and s[0, 0] == np.float32(1e-12) and s[1, 0] == np.float32(1e-12)
    assert (q[:, 0] == 0).all() and q[150, 1] == 127 and s[1, 1] == np.float32(2.0) / np.float32(127.0)


def test_round_trip_is_within_half_a_step_and_rounds_half_away(ora):
    rng = np.random.default_rng(4)
    w = (rng.standard_normal((384, 17)) * np.exp2(rng.integers(-8, 3, size=(384, 17)))).astype(np.float32)
    gs = 128
    q, s = ora.absmax_per_group_symmetric(w, gs)
    s_full = np.repeat(s, gs, axis=0)[:384]
    assert np.abs(q.astype(np.float64) * s_full - w).max() <= 0.5000001 * s_full.max()
    assert (np.abs(q.astype(np.float64) * s_full - w) <= 0.5000001 * s_full).all()
    assert np.abs(q).max() == 127
    w2 = np.array([[127.0], [0.5], [-0.5], [1.5], [-2.5]], dtype=np.float32)   # scale exactly 1
    q2, s2 = ora.absmax_per_group_symmetric(w2, 8)
    assert s2[0, 0] == 1.0 and q2[:, 0].tolist() == [127, 1, -1, 2, -3]


def test_per_group_dequant_to_bf16_truncates(ora):
    """int8_to_bf16.cu:91-110: bf16 bits = upper half of the f32 product, no rounding."""
    q = np.array([[3], [-7]], dtype=np.int8)
    s = np.array([[0.3]], dtype=np.float32)
    bits = ora.int8_to_bf16_per_group(q, s, 2)
    want = ((q.astype(np.float32) * s).view(np.uint32) >> 16).astype(np.uint16)
    assert np.array_equal(bits, want)


# ---- the library's row-major quantiser against the oracle -------------------------------------
@pytest.mark.parametrize("rows,cols,gs", [(5, 256, 128), (3, 200, 64), (7, 64, 64), (2, 130, 128)])
def test_library_quantiser_equals_the_oracle_on_the_transpose(ora, rows, cols, gs):
    rng = np.random.default_rng(rows * cols)
    w = (rng.standard_normal((rows, cols)) * np.exp2(rng.integers(-6, 2, size=(rows, cols)))).astype(np.float32)
    w[0, : min(cols, gs)] = 0.0
    q, s = capi.quantize_per_group_i8(w, gs)
    oq, osc = ora.absmax_per_group_symmetric(np.ascontiguousarray(w.T), gs)   # [K, N] = w transposed
    assert np.array_equal(q, oq.T) and np.array_equal(s.view(np.int32), osc.T.view(np.int32))


# ---- the layer on the GPU ---------------------------------------------------------------------
@pytest.mark.gpu
@pytest.mark.parametrize("gs", [64, 128])
@pytest.mark.parametrize("T", [1, 16, 33, 150, 700])
def test_per_group_layer_against_oracle_on_dequantised_weights(ora, T, gs):
    d, f = 384, 640
    W = S.make_weights(60 + T, 8, d, f, f_s=256, gated=True, router_std=1.0 / np.sqrt(d), outlier_frac=0.002)
    oL, gL = S.build_pair(ora, W, 2, capi.CONVENTION_HUGGINGFACE_QWEN, capi.WEIGHT_INT8_PER_GROUP,
                          group_size=gs)
    x = S.make_tokens(70 + T, T, d)
    with gL:
        out = gL.forward(x)
        idx = gL.last_routing(T)[0]
        o_out, o_idx, _ = oL.execute(x)
        assert np.array_equal(idx, o_idx)
        assert S.rel_err(out, o_out) <= 1e-2


def test_per_group_localises_element_outliers():
    """Why the reference moved from one scale per channel to one per group
    (src/tensor/quantizer.rs:156-165): a single large element coarsens only its own group."""
    rng = np.random.default_rng(7)
    w = rng.standard_normal((64, 1024)).astype(np.float32) * 0.02
    w[np.arange(64), rng.integers(0, 1024, size=64)] *= 40.0   # one outlier per row
    q_r, s_r = capi.quantize_per_row_i8(w)
    q_g, s_g = capi.quantize_per_group_i8(w, 128)
    err_row = np.sqrt(np.mean((q_r * s_r[:, None] - w) ** 2))
    err_grp = np.sqrt(np.mean((q_g * np.repeat(s_g, 128, axis=1) - w) ** 2))
    assert err_grp < 0.5 * err_row, (err_grp, err_row)


@pytest.mark.gpu
def test_per_group_argument_errors(ora):
    W = S.make_weights(1, 4, 128, 128)
    q = {n: capi.quantize_per_group_i8(W[n], 128) for n in ("w_gate", "w_up", "w_down")}
    kw = dict(w_router=W["w_router"], top_k=2, w_gate=q["w_gate"][0], w_up=q["w_up"][0], w_down=q["w_down"][0],
              scale_gate=q["w_gate"][1], scale_up=q["w_up"][1], scale_down=q["w_down"][1],
              weight_dtype=capi.WEIGHT_INT8_PER_GROUP)
    for bad in (0, 96):
        with pytest.raises(capi.MoeHipError) as e:
            capi.Layer(group_size=bad, **kw)
        assert e.value.rc == -1
    capi.Layer(group_size=128, **kw).close()
