"""Expert arithmetic of f32 layers under the reference's NumericPolicy
(src/moe/numeric_policy.rs:36-75, src/moe/dense.rs:120-168): Strict / Fast accumulate the three
projections in f32 (product and sum rounded separately, columns ascending), Certified in f64; the
router is f64 under every policy.  The oracle restates both arithmetics (`policy=STRICT` pinned by
its own known-answer tests), so the f32-accumulating result is compared bit for bit."""
import numpy as np
import pytest

from ateniaengine_amd import capi
from tests import synth as S

pytestmark = pytest.mark.gpu


def _ulp_diff(a, b):
    ai = a.view(np.int32).astype(np.int64)
    bi = b.view(np.int32).astype(np.int64)
    ai = np.where(ai < 0, -(ai & 0x7fffffff), ai)
    bi = np.where(bi < 0, -(bi & 0x7fffffff), bi)
    return np.abs(ai - bi)


@pytest.mark.parametrize("E,k,d,f,fs,gated,T", [
    (4, 2, 64, 96, 0, False, 9),
    (8, 2, 100, 130, 0, False, 33),       # neither dimension a multiple of the 32-wide tiles
    (6, 3, 128, 160, 192, True, 40),      # shared expert with sigmoid gate follows the policy too
    (8, 2, 256, 1024, 0, False, 3),       # long down-projection sums
])
def test_strict_and_fast_accumulate_in_f32(ora, E, k, d, f, fs, gated, T):
    W = S.make_weights(500 + d, E, d, f, f_s=fs, gated=gated, w_std=0.05, router_std=1.0 / np.sqrt(d))
    conv = capi.CONVENTION_HUGGINGFACE_QWEN if fs else capi.CONVENTION_ATENIA
    oL, gL = S.build_pair(ora, W, k, conv, capi.WEIGHT_F32)
    x = S.make_tokens(77, T, d, bf16=False)
    want_cert, o_idx, o_w = oL.execute(x, policy=ora.CERTIFIED)
    want_strict, s_idx, _ = oL.execute(x, policy=ora.STRICT)
    assert (o_idx == s_idx).all()
    assert np.abs(want_cert - want_strict).max() > 0, "the case does not tell the arithmetics apart"
    with gL:
        cert = gL.forward(x).reshape(T, d).copy()
        assert S.rel_err(cert, want_cert) <= 1e-5
        for pol in (capi.POLICY_STRICT, capi.POLICY_FAST):
            gL.set_numeric_policy(pol)
            got = gL.forward(x).reshape(T, d)
            idx, w, *_ = gL.last_routing(T)
            assert (idx == o_idx).all(), "routing must not move with the policy"
            assert _ulp_diff(w, o_w).max() <= 1
            ulps = _ulp_diff(got, want_strict.reshape(T, d))
            # bit for bit except where the device's f64 exp inside silu differs in its last place,
            # which moves one f32 of h by an ulp and the sums that contain it
            assert (ulps > 0).mean() <= 2e-3, f"{(ulps > 0).mean():.2e} of the elements differ"
            assert S.rel_err(got, want_strict) <= 2e-7
            # and it is not simply the f64 result
            assert np.abs(got - cert).max() > 0
        gL.set_numeric_policy(capi.POLICY_CERTIFIED)
        again = gL.forward(x).reshape(T, d)
        assert again.tobytes() == cert.tobytes()


def test_policy_is_accepted_and_ignored_by_blocked_layers(ora):
    """bf16 / int8 layers multiply on the matrix cores with f32 accumulation whatever the policy."""
    W = S.make_weights(9, 8, 128, 256)
    for wd in (capi.WEIGHT_BF16, capi.WEIGHT_INT8_W8A16):
        _, gL = S.build_pair(ora, W, 2, capi.CONVENTION_ATENIA, wd)
        x = S.make_tokens(3, 5, 128)
        with gL:
            a = gL.forward(x).copy()
            gL.set_numeric_policy(capi.POLICY_STRICT)
            b = gL.forward(x).copy()
            assert a.tobytes() == b.tobytes()


def test_unknown_policy_is_rejected(ora):
    W = S.make_weights(9, 4, 32, 48)
    _, gL = S.build_pair(ora, W, 2, capi.CONVENTION_ATENIA, capi.WEIGHT_F32)
    with gL:
        with pytest.raises(capi.MoeHipError) as e:
            gL.set_numeric_policy(7)
        assert e.value.rc == capi.ERR_DIM and "unknown numeric policy 7" in str(e.value)
