"""Pins the oracle's DeepSeek-V3 router: the known-answer cases of the reference's own unit
tests (src/moe/v3_router.rs:340-462, same inputs, same assertions) and the HuggingFace f64
fixture v3_route_ref (tests/moe_v3_route_scale_cert_test.rs:56-175: selected expert sets,
dense combine weights, block output for 6 tokens)."""
import math

import numpy as np
import pytest

from tests import golden_io as G


def sig(x):
    return 1.0 / (1.0 + math.exp(-x))


def test_selects_topk_within_topk_groups(ora):
    idx, w, dense, _ = ora.v3_route([0.0, 0.1, 3.0, 3.1, 0.2, 0.3, 2.5, 2.6], [0.0] * 8, 2, 4, 2)
    assert idx.tolist() == [2, 3]
    assert [(v != 0.0) for v in dense] == [i in (2, 3) for i in range(8)]


def test_bias_changes_selection_not_combine_weight(ora):
    logits = [0.0, 0.0, 1.0, 1.05, 0.0, 0.0, 1.0, 0.9]
    no_bias = ora.v3_route(logits, [0.0] * 8, 2, 4, 2)
    bias = [0.0] * 7 + [0.5]
    idx, w, _, _ = ora.v3_route(logits, bias, 2, 4, 2)
    assert no_bias[0].tolist() != idx.tolist()
    assert 7 in idx.tolist()
    raw = [sig(float(np.float32(logits[i]))) for i in idx]
    slot = idx.tolist().index(7)
    assert abs(float(w[slot]) - sig(float(np.float32(0.9))) / sum(raw)) < 1e-6


def test_scaling_and_normalisation(ora):
    logits = [0.2, 0.4, 2.0, 2.1, 0.1, 0.0, 1.8, 1.9]
    a = ora.v3_route(logits, [0.0] * 8, 2, 4, 2, 1.0)
    b = ora.v3_route(logits, [0.0] * 8, 2, 4, 2, 2.5)
    assert a[0].tolist() == b[0].tolist()
    assert np.abs(b[1] - a[1] * 2.5).max() < 1e-5
    logits = [0.0, 0.0, 2.0, 2.2, 0.0, 0.0, 1.5, 1.7]
    r = ora.v3_route(logits, [0.0] * 8, 2, 4, 2, 1.0, True)
    assert abs(float(r[1].sum()) - 1.0) < 1e-5
    raw = ora.v3_route(logits, [0.0] * 8, 2, 4, 2, 1.0, False)
    assert abs(float(raw[1][raw[0].tolist().index(3)]) - sig(float(np.float32(2.2)))) < 1e-6


def test_group_limiting_excludes_the_largest_single_expert(ora):
    idx, *_ = ora.v3_route([5.0, -5.0, 1.0, 1.0, 1.0, 1.0, -5.0, -5.0], [0.0] * 8, 2, 4, 2)
    assert 0 not in idx.tolist() and all(2 <= i < 6 for i in idx)
    assert idx.tolist() == [2, 3]  # all four candidates tie: the lower indices win


def test_ties_between_groups_go_to_the_lower_group(ora):
    idx, *_ = ora.v3_route([1.0] * 8, [0.0] * 8, 3, 4, 2)
    assert idx.tolist() == [0, 1, 2]


def test_margin_is_min_selected_minus_max_unselected_in_groups(ora):
    logits = [0.3, 0.4, 1.1, 1.2, 0.9, 0.8, 1.5, 1.6]
    bias = [0.05, 0.0, 0.1, 0.0, 0.0, 0.2, 0.0, 0.0]
    idx, w, dense, margin = ora.v3_route(logits, bias, 3, 4, 2, 2.5)
    again = ora.v3_route(logits, bias, 3, 4, 2, 2.5)
    assert idx.tolist() == again[0].tolist() and w.tobytes() == again[1].tobytes()
    choice = [sig(float(np.float32(l))) + float(np.float32(b)) for l, b in zip(logits, bias)]
    assert idx.tolist() == [2, 6, 7]  # groups 1 and 3; experts 7, 6 and 2 (1.1 + bias 0.1)
    assert margin == pytest.approx(min(choice[i] for i in idx) - choice[3], abs=1e-15)
    all_in = ora.v3_route(logits, bias, 4, 4, 2)
    assert all_in[3] == math.inf


def test_fail_loud(ora):
    def rc(*a, **k):
        with pytest.raises(ora.OracleError) as e:
            ora.v3_route(*a, **k)
        return e.value.rc, e.value.index

    z = lambda n: [0.0] * n
    assert rc(z(7), z(7), 2, 4, 2)[0] == ora.V3_ERR_NOT_DIVISIBLE
    assert rc(z(4), z(4), 1, 4, 2) == (ora.V3_ERR_GROUP_TOO_SMALL, 1)
    assert rc(z(8), z(8), 2, 4, 5)[0] == ora.V3_ERR_TOPK_GROUP_EXCEEDS
    assert rc(z(8), z(8), 5, 4, 2) == (ora.V3_ERR_TOPK_EXCEEDS, 4)
    assert rc(z(6), z(8), 2, 4, 2)[0] == ora.ERR_DIM
    assert rc([float("nan")] * 8, z(8), 2, 4, 2) == (ora.V3_ERR_NON_FINITE_LOGIT, 0)
    assert rc(z(8), z(5) + [float("inf")] + z(2), 2, 4, 2) == (ora.V3_ERR_NON_FINITE_BIAS, 5)
    assert rc(z(8), z(8), 0, 4, 2) == (ora.V3_ERR_ZERO_PARAMETER, 0)
    assert rc(z(8), z(8), 2, 0, 2) == (ora.V3_ERR_ZERO_PARAMETER, 1)
    assert rc(z(8), z(8), 2, 4, 0) == (ora.V3_ERR_ZERO_PARAMETER, 2)


def test_hf_fixture_sets_weights_and_block(ora):
    j, t = G.sidecar("v3_route_ref"), G.tensors("v3_route_ref")
    n, k, d = j["n_routed_experts"], j["top_k"], j["hidden_size"]
    L = G.v3_oracle_layer(ora)
    hidden = t["hidden"]
    out, idx, w = L.v3_forward(hidden, t["router.bias"], j["n_group"], j["topk_group"],
                               j["routed_scaling_factor"], j["norm_topk_prob"])
    assert idx.tolist() == j["selected_experts"]
    dense = np.zeros((j["tokens"], n))
    for tok in range(j["tokens"]):
        dense[tok, idx[tok]] = w[tok]
    ref_dense = np.array(j["dense_combine_weights"]).reshape(j["tokens"], n)
    assert np.abs(dense - ref_dense).max() < 1e-6      # the reference's gate is 1e-3
    ref_block = np.array(j["block_out"]).reshape(j["tokens"], d)
    assert np.abs(out - ref_block).max() < 1e-6
    # the margins the fixture records come from the same choice values
    for tok in range(j["tokens"]):
        logits = ora.matvec(t["router.weight"], hidden[tok])
        m = ora.v3_route(logits, t["router.bias"], k, j["n_group"], j["topk_group"],
                         j["routed_scaling_factor"], j["norm_topk_prob"])[3]
        assert m == pytest.approx(j["selection_margins"][tok], abs=1e-5)
