"""Known-answer tests that pin the CPU oracle to the reference's own unit tests.

Each case restates an assertion of the reference's in-module tests (cited), so a
dropped term, wrong sign, wrong tie-break or transposed operand in the oracle fails here.
"""
import math

import numpy as np
import pytest


# ---- sparse.rs:294-339 (top-k KATs) -----------------------------------------------------
def test_top_k_selects_largest(ora):
    idx, _ = ora.top_k_routing_with([0.1, 0.5, 0.2, 0.4], 2)
    assert idx.tolist() == [1, 3]


def test_top_k_tie_breaks_by_lower_index(ora):
    idx, _ = ora.top_k_routing_with([0.25, 0.25, 0.25, 0.25], 2)
    assert idx.tolist() == [0, 1]


def test_top_k_errors(ora):
    with pytest.raises(ora.OracleError) as e:
        ora.top_k_routing_with([0.5, 0.5], 0)
    assert e.value.rc == ora.ERR_ZERO_K
    with pytest.raises(ora.OracleError) as e:
        ora.top_k_routing_with([0.5, 0.5], 3)
    assert e.value.rc == ora.ERR_K_EXCEEDS
    with pytest.raises(ora.OracleError) as e:
        ora.top_k_routing_with([0.5, float("nan"), 0.5], 2)
    assert (e.value.rc, e.value.index) == (ora.ERR_NON_FINITE, 1)
    with pytest.raises(ora.OracleError) as e:
        ora.top_k_routing_with([0.5, -0.1], 1)
    assert (e.value.rc, e.value.index) == (ora.ERR_NEGATIVE, 1)
    with pytest.raises(ora.OracleError) as e:
        ora.top_k_routing_with([0.0, 0.0], 1)
    assert e.value.rc == ora.ERR_SUM_NON_POSITIVE


def test_top_k_renormalised(ora):
    idx, w = ora.top_k_routing_with([0.1, 0.6, 0.3], 2)
    assert idx.tolist() == [1, 2]
    assert abs(float(w.sum()) - 1.0) < 1e-6
    assert abs(w[0] - 0.6 / 0.9) < 1e-5 and abs(w[1] - 0.3 / 0.9) < 1e-5
    # exact cast sequence: (f32)((f64)w * (1/sum_f64))
    s = float(np.float32(0.6)) + float(np.float32(0.3))
    assert w[0] == np.float32(float(np.float32(0.6)) * (1.0 / s))


def test_top_k_no_renorm_keeps_raw(ora):
    idx, w = ora.top_k_routing_with([0.1, 0.6, 0.3], 2, renormalize=False)
    assert idx.tolist() == [1, 2]
    assert w.tolist() == [np.float32(0.6), np.float32(0.3)]


def test_top_k_against_bruteforce_sort(ora):
    rng = np.random.default_rng(0)
    for _ in range(300):
        n = int(rng.integers(1, 70))
        k = int(rng.integers(1, n + 1))
        w = rng.random(n).astype(np.float32)
        if rng.random() < 0.5:  # engineered ties
            w[rng.integers(0, n, size=n // 2 + 1)] = w[0]
        order = sorted(range(n), key=lambda i: (-float(w[i]), i))
        idx, _ = ora.top_k_routing_with(w, k, renormalize=False)
        assert idx.tolist() == sorted(order[:k])


# ---- dense.rs:457-464, 591-602 (softmax) ------------------------------------------------
def test_softmax_sums_to_one_and_closed_form(ora):
    w = ora.softmax([1.0, 2.0, 3.0])
    assert abs(float(w.sum()) - 1.0) < 1e-6
    e = [math.exp(-2.0), math.exp(-1.0), 1.0]
    s = e[0] + e[1] + e[2]
    assert w.tolist() == [np.float32(v * (1.0 / s)) for v in e]
    u = ora.softmax([5.0] * 8)
    assert u.tolist() == [np.float32(0.125)] * 8
    # shift invariance holds exactly when the shifted logits are exact in f32
    a = ora.softmax([0.5, -1.25, 2.0, 0.0])
    b = ora.softmax([0.5 + 64, -1.25 + 64, 2.0 + 64, 64.0])
    assert a.tolist() == b.tolist()


def test_softmax_subtracts_in_f32(ora):
    # max = 1e8 (f32). (v - max) in f32 differs from the f64 difference for v = 3.0:
    # f32(3 - 1e8) = -1e8 exactly (ulp 8), so exp underflows identically for 3.0 and 0.0.
    w = ora.softmax([1e8, 3.0, 0.0])
    assert w.tolist() == [1.0, 0.0, 0.0]
    big = np.float32(16777216.0)  # 2^24: big - 1 is not representable + 1 ulp games
    lo = np.float32(16777215.0)
    w = ora.softmax([big, lo])
    d = float(np.float32(lo - big))
    e = math.exp(d)
    s = 1.0 + e
    assert w.tolist() == [np.float32(1.0 * (1.0 / s)), np.float32(e * (1.0 / s))]


def test_softmax_nan_surfaces_as_non_finite(ora):
    w = ora.softmax([0.0, float("nan"), 1.0])
    assert math.isnan(w[1])
    with pytest.raises(ora.OracleError) as e:
        ora.top_k_routing_with(w, 2)
    assert (e.value.rc, e.value.index) == (ora.ERR_NON_FINITE, 1)


# ---- dense.rs:74-77, 97-135 --------------------------------------------------------------
def test_silu_values(ora):
    assert ora.silu(0.0) == 0.0
    for v in (-3.0, -0.5, 0.25, 1.0, 7.5):
        assert ora.silu(v) == np.float32(v / (1.0 + math.exp(-v)))
    assert ora.silu(1.0) > 0 > ora.silu(-1.0)


def test_matvec_f64_accumulation_order_and_orientation(ora):
    # W is [rows, cols]; a transposed read would fail the non-square case.
    w = np.arange(6, dtype=np.float32).reshape(2, 3)
    x = np.array([1.0, 10.0, 100.0], dtype=np.float32)
    assert ora.matvec(w, x).tolist() == [210.0, 543.0]
    # f64 accumulation keeps what f32 accumulation loses.
    w = np.array([[1e8, 1.0, -1e8]], dtype=np.float32)
    x = np.ones(3, dtype=np.float32)
    assert ora.matvec(w, x).tolist() == [1.0]
    assert ora.matvec(w, x, f32acc=True).tolist() == [0.0]
    # sequential c-ascending f64 sum, bit for bit
    rng = np.random.default_rng(1)
    w = rng.standard_normal((5, 777)).astype(np.float32)
    x = rng.standard_normal(777).astype(np.float32)
    exp = []
    for r in range(5):
        acc = 0.0
        for c in range(777):
            acc += float(w[r, c]) * float(x[c])
        exp.append(np.float32(acc))
    assert ora.matvec(w, x).tolist() == exp


def test_matvec_threads_do_not_change_bits(ora):
    rng = np.random.default_rng(2)
    w = rng.standard_normal((512, 256)).astype(np.float32)  # above the 65536 threshold
    x = rng.standard_normal(256).astype(np.float32)
    ora.set_threads(1)
    a = ora.matvec(w, x)
    ora.set_threads(4)
    b = ora.matvec(w, x)
    ora.set_threads(1)
    assert a.tobytes() == b.tobytes()


# ---- dense.rs:368-406 synthetic fixture layer + invariants (dense.rs:467-519,
#      sparse.rs:342-386) ------------------------------------------------------------------
def _seeded_py(seed, n):
    state = (seed * 0x9E3779B97F4A7C15 + 1) & 0xFFFFFFFFFFFFFFFF
    out = []
    for _ in range(n):
        state ^= (state << 13) & 0xFFFFFFFFFFFFFFFF
        state ^= state >> 7
        state ^= (state << 17) & 0xFFFFFFFFFFFFFFFF
        u = (state >> 11) & 0xFFFFFFFF
        out.append(np.float32(np.float32(np.float32(u) / np.float32(0xFFFFFFFF)) * np.float32(2.0))
                   - np.float32(1.0))
    return np.array(out, dtype=np.float32)


def test_seeded_matches_restated_xorshift(ora):
    for seed in (1, 7, 1011, 1033):
        a = ora.seeded(seed, 200)
        assert a.tobytes() == _seeded_py(seed, 200).tobytes()
        assert a.min() >= -1.0 and a.max() <= 1.0


def build_fixture_layer(ora, top_k=2, convention=0):
    d, f, E = 8, 16, 4
    return ora.Layer(
        w_router=ora.seeded(1, E * d).reshape(E, d),
        w_gate=np.stack([ora.seeded((100 + e) * 10 + 1, f * d).reshape(f, d) for e in range(E)]),
        w_up=np.stack([ora.seeded((100 + e) * 10 + 2, f * d).reshape(f, d) for e in range(E)]),
        w_down=np.stack([ora.seeded((100 + e) * 10 + 3, d * f).reshape(d, f) for e in range(E)]),
        top_k=top_k, convention=convention)


def test_sparse_matches_dense_restricted_and_manual_sum(ora):
    L = build_fixture_layer(ora)
    x = ora.seeded(7, L.d)
    out, idx, w = L.forward_with(x)
    _, sm = L.route(x)
    assert idx.tolist() == ora.top_k_routing_with(sm, 2)[0].tolist()
    ys = np.concatenate([ora.expert_forward(L.w_gate[e], L.w_up[e], L.w_down[e], x)
                         for e in range(L.E)])
    manual = ora.combine_selected(idx, w, ys, L.d)
    assert out.tobytes() == manual.tobytes()
    # dense-restricted oracle (sparse.rs:243-268): renormalise over the given subset
    s = sum(float(sm[e]) for e in idx)
    exp = np.zeros(L.d, dtype=np.float32)
    for e in idx:
        we = np.float32(float(sm[e]) * (1.0 / s))
        exp = exp + we * ys[e * L.d:(e + 1) * L.d]
    assert np.abs(out - exp).max() < 1e-5


def test_k_all_equals_dense_forward(ora):
    L = build_fixture_layer(ora, top_k=4)
    x = ora.seeded(11, L.d)
    out, idx, _ = L.forward_with(x)
    assert idx.tolist() == [0, 1, 2, 3]
    _, sm = L.route(x)
    dense = np.zeros(L.d, dtype=np.float32)
    for e in range(L.E):
        dense = dense + sm[e] * ora.expert_forward(L.w_gate[e], L.w_up[e], L.w_down[e], x)
    assert np.abs(out - dense).max() < 1e-5


def test_identical_experts_collapse_to_one(ora):
    L = build_fixture_layer(ora)
    for a in (L.w_gate, L.w_up, L.w_down):
        a[:] = a[0]
    x = ora.seeded(5, L.d)
    out, _, w = L.forward_with(x)
    one = ora.expert_forward(L.w_gate[0], L.w_up[0], L.w_down[0], x)
    assert abs(float(w.sum()) - 1.0) < 1e-6
    assert np.abs(out - one).max() < 1e-5


def test_determinism_and_batch_rows_independent(ora):
    L = build_fixture_layer(ora)
    xs = np.stack([ora.seeded(20 + t, L.d) for t in range(5)])
    out, idx, w = L.execute(xs)
    for t in range(5):
        o1, i1, w1 = L.forward_with(xs[t])
        assert o1.tobytes() == out[t].tobytes() and i1.tolist() == idx[t].tolist()
        assert w1.tobytes() == w[t].tobytes()
    assert np.isfinite(out).all()


def test_policies_agree_within_tolerance(ora):
    L = build_fixture_layer(ora)
    x = ora.seeded(3, L.d)
    a, _, _ = L.forward_with(x, policy=ora.CERTIFIED)
    b, _, _ = L.forward_with(x, policy=ora.STRICT)
    assert np.abs(a - b).max() < 1e-4


def test_sigmoid_dot(ora):
    assert ora.sigmoid_dot([0.0, 0.0], [1.0, 2.0]) == 0.5
    g, x = [0.5, -1.5, 2.0], [1.0, 2.0, 0.25]
    acc = 0.5 * 1.0 + (-1.5) * 2.0 + 2.0 * 0.25
    assert ora.sigmoid_dot(g, x) == np.float32(1.0 / (1.0 + math.exp(-acc)))


# ---- disk_tier.rs:1309-1334, quantizer.rs:969-993,1050-1062 ------------------------------
def test_quantize_per_row(ora):
    rng = np.random.default_rng(3)
    w = (rng.standard_normal((7, 33)) * 0.02).astype(np.float32)
    w[3] = 0.0
    q, s = ora.quantize_per_row_i8(w)
    assert s[3] == 1.0 and (q[3] == 0).all()
    dq = ora.dequantize_per_row_i8(q, s)
    amax = np.abs(w).max(axis=1)
    assert (np.abs(dq - w).max(axis=1) <= amax / 254 * (1 + 1e-5) + 1e-12).all()
    assert (np.abs(q).max(axis=1)[amax > 0] == 127).all()
    # half away from zero: row amax = 127 => scale 1 => q = round(w)
    q, s = ora.quantize_per_row_i8(np.array([[127.0, 0.5, -0.5, 1.5, -2.5]], dtype=np.float32))
    assert s[0] == 1.0 and q[0].tolist() == [127, 1, -1, 2, -3]


def test_absmax_per_channel_and_bf16_dequant(ora):
    q, s = ora.absmax_per_channel_symmetric(np.array([[2.0], [-4.0], [6.0], [-127.0]]))
    assert s.tolist() == [1.0] and q[:, 0].tolist() == [2, -4, 6, -127]
    q, s = ora.absmax_per_channel_symmetric(np.zeros((3, 2)))
    assert s.tolist() == [np.float32(1e-12)] * 2 and (q == 0).all()
    rng = np.random.default_rng(4)
    w = rng.standard_normal((16, 5)).astype(np.float32)
    q, s = ora.absmax_per_channel_symmetric(w)
    b = ora.int8_to_bf16_per_channel(q, s)
    exp = ((q.astype(np.float32) * s[None, :]).view(np.uint32) >> 16).astype(np.uint16)
    assert (b == exp).all()


# ---- tensor.rs:294-308, residency.rs:1487-1500 -------------------------------------------
def test_bf16_truncation_roundtrip(ora):
    lib = ora.lib()
    assert lib.ora_f32_to_bf16_bits(1.0) == 0x3F80
    assert lib.ora_bf16_bits_to_f32(0x3F80) == 1.0
    # truncation, not rounding: 1 + 2^-8 + 2^-9 truncates down to 1.0
    assert lib.ora_f32_to_bf16_bits(1.0 + 2.0**-8 + 2.0**-9) == 0x3F80
    a = np.random.default_rng(5).standard_normal(1000).astype(np.float32)
    b = ora.f32_to_bf16_bits(a)
    up = ora.bf16_bits_to_f32(b)
    assert (ora.f32_to_bf16_bits(up) == b).all()
    assert (np.abs(up) <= np.abs(a)).all()


# ---- derived permutation contract vs brute force -----------------------------------------
def test_permute_vs_bruteforce(ora):
    rng = np.random.default_rng(6)
    for (T, k, E) in [(1, 2, 8), (5, 2, 4), (64, 4, 60), (33, 6, 64), (7, 1, 3)]:
        idx = np.stack([np.sort(rng.choice(E, size=k, replace=False)) for _ in range(T)])
        if T == 5:
            idx[:] = [1, 3]  # empty experts 0, 2
        counts, offsets, perm = ora.permute(idx.astype(np.int32), E)
        flat = idx.reshape(-1)
        exp_perm = [p for e in range(E) for p in range(T * k) if flat[p] == e]
        assert perm.tolist() == exp_perm
        assert counts.tolist() == [int((flat == e).sum()) for e in range(E)]
        assert offsets.tolist() == [0] + np.cumsum(counts).tolist()


def test_numerical_metrics(ora):
    m = ora.numerical_metrics([1.0, 2.0, 4.0], [1.5, 2.0, 3.0])
    assert m["max_abs_diff"] == 1.0 and m["mean_abs_diff"] == 0.5
    assert abs(m["rmse"] - math.sqrt((0.25 + 1.0) / 3)) < 1e-15 and m["argmax_match"]
    assert not ora.numerical_metrics([3.0, 1.0], [1.0, 3.0])["argmax_match"]
