"""DeepSeek-V3 routing on the GPU (atenia_moe_hip_layer_set_v3_router) against the oracle's
restatement of src/moe/v3_router.rs and the HuggingFace f64 fixture v3_route_ref."""
import numpy as np
import pytest

from ateniaengine_amd import capi
from tests import golden_io as G
from tests import synth as S

pytestmark = pytest.mark.gpu


def _ulp(a, b):
    ia = np.ascontiguousarray(a, np.float32).view(np.int32).astype(np.int64)
    ib = np.ascontiguousarray(b, np.float32).view(np.int32).astype(np.int64)
    return np.abs(ia - ib)


def _oracle_routes(ora, oL, x, bias, k, n_group, topk_group, scale, norm):
    idx, w = [], []
    for row in x:
        i, ww, _, _ = ora.v3_route(ora.matvec(oL.w_router, row), bias, k, n_group, topk_group, scale, norm)
        idx.append(i)
        w.append(ww)
    return np.stack(idx), np.stack(w)


def test_hf_fixture_on_device(ora):
    j, t = G.sidecar("v3_route_ref"), G.tensors("v3_route_ref")
    a = G.v3_arrays()
    with capi.Layer(top_k=j["top_k"], convention=capi.CONVENTION_HUGGINGFACE_QWEN,
                    weight_dtype=capi.WEIGHT_F32, **a) as gL:
        gL.set_v3_router(j["n_group"], j["topk_group"], j["routed_scaling_factor"], j["norm_topk_prob"],
                         t["router.bias"])
        out = gL.forward(t["hidden"])
        idx, w = gL.last_routing(j["tokens"])[:2]
        assert idx.tolist() == j["selected_experts"]
        n = j["n_routed_experts"]
        dense = np.zeros((j["tokens"], n))
        for tok in range(j["tokens"]):
            dense[tok, idx[tok]] = w[tok]
        assert np.abs(dense - np.array(j["dense_combine_weights"]).reshape(-1, n)).max() < 1e-6
        ref = np.array(j["block_out"]).reshape(j["tokens"], -1)
        assert np.abs(out - ref).max() < 1e-6
        o_out, o_idx, o_w = G.v3_oracle_layer(ora).v3_forward(
            t["hidden"], t["router.bias"], j["n_group"], j["topk_group"], j["routed_scaling_factor"],
            j["norm_topk_prob"])
        assert np.array_equal(idx, o_idx) and _ulp(w, o_w).max() <= 1
        assert S.rel_err(out, o_out) <= 1e-6


V3_CASES = [
    # E, k, n_group, topk_group, d, T, scale, norm, wd
    (256, 8, 8, 4, 512, 1, 2.5, True, capi.WEIGHT_BF16),
    (256, 8, 8, 4, 512, 37, 2.5, True, capi.WEIGHT_BF16),
    (256, 8, 8, 4, 512, 1500, 2.5, True, capi.WEIGHT_BF16),
    (60, 4, 6, 3, 256, 300, 1.0, False, capi.WEIGHT_F32),
    (64, 6, 8, 3, 128, 700, 16.0, True, capi.WEIGHT_INT8_W8A16),
    (8, 2, 4, 2, 64, 19, 1.0, True, capi.WEIGHT_F32),
    (160, 6, 8, 3, 320, 70, 16.0, False, capi.WEIGHT_BF16),
]


@pytest.mark.parametrize("E,k,n_group,topk_group,d,T,scale,norm,wd", V3_CASES)
def test_v3_routing_bit_exact(ora, E, k, n_group, topk_group, d, T, scale, norm, wd):
    W = S.make_weights(E + T, E, d, 16, f_s=16, router_std=1.5 / np.sqrt(d))
    oL, gL = S.build_pair(ora, W, k, capi.CONVENTION_HUGGINGFACE_QWEN, wd)
    bias = (0.05 * np.random.default_rng(E).standard_normal(E)).astype(np.float32)
    x = S.make_tokens(7 * E + T, T, d, bf16=wd != capi.WEIGHT_F32)
    with gL:
        gL.set_v3_router(n_group, topk_group, scale, norm, bias)
        idx, w = gL.route(x)
        o_idx, o_w = _oracle_routes(ora, oL, x, bias, k, n_group, topk_group, scale, norm)
        assert (idx == o_idx).all(), f"{(idx != o_idx).any(axis=1).sum()} tokens routed differently"
        assert _ulp(w, o_w).max() <= 1
        n = min(T, 12)  # whole layer on a few rows: combine and ungated shared expert included
        out = gL.forward(x[:n])
        o_out = oL.v3_forward(x[:n], bias, n_group, topk_group, scale, norm)[0]
        tol = 1e-5 if wd == capi.WEIGHT_F32 else 2e-2
        assert S.rel_err(out, o_out) <= tol


def test_v3_ties_go_to_lower_group_and_lower_index(ora):
    E, k, d = 16, 3, 64
    W = S.make_weights(1, E, d, 16)
    W["w_router"][:] = W["w_router"][0]  # all logits equal for every token
    oL, gL = S.build_pair(ora, W, k, capi.CONVENTION_HUGGINGFACE_QWEN, capi.WEIGHT_F32)
    with gL:
        gL.set_v3_router(4, 2, 1.0, True, np.zeros(E, np.float32))
        idx, w = gL.route(S.make_tokens(2, 5, d, bf16=False))
        assert (idx == np.array([0, 1, 2])).all()
        assert np.allclose(w, 1.0 / 3.0, atol=1e-7)
        bias = np.zeros(E, np.float32)
        bias[13] = 0.25  # lifts group 3 and expert 13 for selection; weights stay the raw scores
        gL.set_v3_router(4, 2, 1.0, True, bias)
        idx, w = gL.route(S.make_tokens(2, 5, d, bf16=False))
        assert (idx == np.array([0, 1, 13])).all()
        assert np.allclose(w, 1.0 / 3.0, atol=1e-7)


def test_v3_configuration_errors_and_non_finite_logit(ora):
    W = S.make_weights(2, 8, 64, 16)
    _, gL = S.build_pair(ora, W, 2, capi.CONVENTION_HUGGINGFACE_QWEN, capi.WEIGHT_F32)
    z = np.zeros(8, np.float32)
    with gL:
        def err(*a):
            with pytest.raises(capi.MoeHipError) as e:
                gL.set_v3_router(*a)
            return e.value.rc, str(e.value)

        assert "n_group must be > 0" in err(0, 2, 1.0, True, z)[1]
        assert "topk_group must be > 0" in err(4, 0, 1.0, True, z)[1]
        assert "n_routed_experts (8) not divisible by n_group (3)" in err(3, 2, 1.0, True, z)[1]
        assert "experts_per_group (1) < 2" in err(8, 2, 1.0, True, z)[1]
        assert "topk_group (5) > n_group (4)" in err(4, 5, 1.0, True, z)[1]
        rc, msg = err(4, 1, 1.0, True, np.where(np.arange(8) == 5, np.inf, 0).astype(np.float32))
        assert rc == -3 and "e_score_correction_bias at 5 is non-finite" in msg
        x = S.make_tokens(3, 4, 64, bf16=False)
        before = gL.forward(x)  # the failed calls left the softmax router in place
        gL.set_v3_router(4, 2, 1.0, True, z)
        assert not np.array_equal(gL.forward(x), before)
        bad = x.copy()
        bad[2, 7] = np.nan
        with pytest.raises(capi.MoeHipError) as e:
            gL.forward(bad)
        assert e.value.rc == -3 and gL.last_non_finite()[0] == 2
        assert np.isfinite(gL.forward(x)).all()
    W3 = S.make_weights(2, 8, 64, 16)
    _, g3 = S.build_pair(ora, W3, 3, capi.CONVENTION_HUGGINGFACE_QWEN, capi.WEIGHT_F32)
    with g3:
        with pytest.raises(capi.MoeHipError) as e:
            g3.set_v3_router(4, 1, 1.0, True, z)
        assert "top_k (3) exceeds experts in selected groups (2)" in str(e.value)
