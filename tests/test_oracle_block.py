"""Pins the oracle's decoder-layer FFN block (RMSNorm * gamma -> MoE -> residual add):
closed forms chosen so that each plausible mistake fails one of them, and the reference's
whole-model fixture with HuggingFace f64 logits (tests/moe_full_forward_test.rs:140-165)."""
import numpy as np
import pytest

from tests import tiny_mixtral as TM


@pytest.mark.parametrize("policy", [0, 1])
def test_norm_3_4_0_0(ora, policy):
    """mla.rs:689-696: mean square of the output is 1 for unit gamma; here the exact values:
    mean(x^2) = 6.25, so y = x / sqrt(6.25 + eps)."""
    eps = 1e-5
    y = ora.rms_norm_gamma([3.0, 4.0, 0.0, 0.0], [1.0] * 4, eps, policy)
    want = np.array([3.0, 4.0, 0.0, 0.0]) / np.sqrt(6.25 + np.float64(np.float32(eps)))
    assert np.abs(y - want).max() <= 2.5e-7  # one f32 rounding of inv, one of the product
    assert abs(float((y.astype(np.float64) ** 2).mean()) - 1.0) < 1e-5


def test_eps_is_inside_the_root(ora):
    """An all-zero row: y = 0 * 1/sqrt(eps) = 0 (finite); a tiny row is scaled by ~1/sqrt(eps),
    which 1/(rms + eps) or 1/sqrt(ms) + eps would not give."""
    for policy in (0, 1):
        assert np.all(ora.rms_norm_gamma([0.0] * 8, [1.0] * 8, 1e-6, policy) == 0.0)
        y = ora.rms_norm_gamma([1e-9] * 4, [1.0] * 4, 1e-6, policy)
        assert np.allclose(y, 1e-9 / np.sqrt(1e-18 + 1e-6), rtol=1e-6)


def test_gamma_is_per_column_and_applied_last(ora):
    x = np.array([1.0, -2.0, 3.0, -4.0], dtype=np.float32)
    g = np.array([0.0, 1.0, -2.0, 0.5], dtype=np.float32)
    for policy in (0, 1):
        base = ora.rms_norm_gamma(x, np.ones(4), 1e-5, policy)
        y = ora.rms_norm_gamma(x, g, 1e-5, policy)
        assert np.array_equal(y, base * g)  # a single f32 product per element, after the norm


def test_f32_policy_sums_left_to_right_in_f32(ora):
    """x = [4096, 1, 1, ..., 1]: 4096^2 = 2^24, and 2^24 + 1 rounds back to 2^24 in f32, so the
    left-to-right f32 sum never sees the ones; with the head last, (n-1) + 2^24 is exact.  The
    f64 policy counts every one in both orders.  A pairwise / vectorised / f64 sum under the f32
    policy, or an f32 sum under the f64 policy, fails this."""
    n, eps = 1025, 0.0
    head_first = np.ones(n, dtype=np.float32)
    head_first[0] = 4096.0
    head_last = head_first[::-1].copy()
    ones = np.ones(n, dtype=np.float32)
    inv = lambda s: np.float32(1.0) / np.sqrt(np.float32(s) / np.float32(n), dtype=np.float32)
    y = ora.rms_norm_gamma(head_first, ones, eps, 0)
    assert y[1] == inv(2.0 ** 24)
    y = ora.rms_norm_gamma(head_last, ones, eps, 0)
    assert y[0] == inv(2.0 ** 24 + 1024)
    assert inv(2.0 ** 24) != inv(2.0 ** 24 + 1024)
    for x in (head_first, head_last):
        y = ora.rms_norm_gamma(x, ones, eps, 1)
        want = 1.0 / np.sqrt((2.0 ** 24 + 1024) / n)
        assert y[x == 1.0][0] == np.float32(want)


def test_f32_policy_rounds_the_normalised_value_before_gamma(ora):
    """Under the f32 policy (v * inv) is rounded to f32 and then multiplied by gamma; folding
    inv * gamma first gives different bits for some elements of a generic row."""
    rng = np.random.default_rng(5)
    x = rng.standard_normal(4096).astype(np.float32)
    g = (1.0 + 0.1 * rng.standard_normal(4096)).astype(np.float32)
    y = ora.rms_norm_gamma(x, g, 1e-5, 0)
    s = np.float32(0.0)
    for v in x:
        s = np.float32(s + np.float32(v * v))
    inv = np.float32(1.0) / np.sqrt(np.float32(s / np.float32(4096.0)) + np.float32(1e-5), dtype=np.float32)
    assert np.array_equal(y, (x * inv) * g)
    assert not np.array_equal(y, x * (inv * g))


def test_block_is_residual_plus_moe_of_normed(ora):
    from tests import synth as S

    W = S.make_weights(3, 4, 16, 24)
    L = ora.Layer(top_k=2, **W)
    rng = np.random.default_rng(0)
    x1 = rng.standard_normal((3, 16)).astype(np.float32)
    g = rng.standard_normal(16).astype(np.float32)
    for policy in (0, 1):
        out, h2, idx, w = L.block_forward(x1, g, 1e-5, policy)
        for t in range(3):
            assert np.array_equal(h2[t], ora.rms_norm_gamma(x1[t], g, 1e-5, policy))
            y, i, ww = L.forward_with(h2[t])
            assert np.array_equal(out[t], x1[t] + y) and i.tolist() == idx[t].tolist()


@pytest.mark.parametrize("policy", [0, 1])
def test_tiny_mixtral_logits_match_hf(ora, policy):
    _, t = TM.load()

    def block(layer, x1, gamma, eps):
        L = ora.Layer(top_k=2, convention=ora.ATENIA, **TM.moe_arrays(t, layer))
        return L.block_forward(x1, gamma, eps, policy)[0]

    got, want = TM.logits(block), TM.hf_logits()
    assert np.abs(got - want).max() < 1e-6  # measured 2.5e-8; the reference's own bar is 1e-3
    assert np.array_equal(got.argmax(-1), want.argmax(-1))


# Topology fixtures of the reference's tests/moe_scale_cert_test.rs: Mixtral with grouped heads
# (8 experts, top-2, renormalised) and Qwen2-MoE (16 experts, top-4 raw weights, sigmoid-gated
# shared expert).  The block's convention is what differs between them.
# DeepSeek-V2: HuggingFace's block multiplies by the raw softmax weights and adds its fused shared
# experts ungated, whatever `norm_topk_prob` says (the case of the reference's deepseek_block
# fixture as well) -- HUGGINGFACE_QWEN without a gate vector.  The reference's runtime renormalises
# for this config (norm_topk_prob = true, src/moe/runtime.rs:894-907) and certifies it under a
# 1e-2 bound (tests/moe_scale_cert_test.rs:105-111); that variant is checked to sit inside that
# bound and outside ours.
SCALE_CONVENTION = {"mixtral_scale": "ATENIA", "qwen_scale": "HUGGINGFACE_QWEN",
                    "deepseek_scale": "HUGGINGFACE_QWEN"}
SCALE_TOL = {"mixtral_scale": 1e-6, "qwen_scale": 1e-6, "deepseek_scale": 1e-6}


@pytest.mark.parametrize("name", TM.SCALE)
@pytest.mark.parametrize("policy", [0, 1])
def test_scale_fixture_logits_match_hf(ora, name, policy):
    cfg, t = TM.load(name)
    conv = getattr(ora, SCALE_CONVENTION[name])

    def block(layer, x1, gamma, eps):
        L = ora.Layer(top_k=TM.top_k(cfg), convention=conv, **TM.moe_arrays(t, layer))
        return L.block_forward(x1, gamma, eps, policy)[0]

    got, want = TM.logits(block, name), TM.hf_logits(name)
    assert np.abs(got - want).max() < SCALE_TOL[name], np.abs(got - want).max()
    assert np.array_equal(got.argmax(-1), want.argmax(-1))


def test_deepseek_scale_renormalised_variant_sits_inside_the_reference_bound(ora):
    cfg, t = TM.load("deepseek_scale")

    def block(layer, x1, gamma, eps):
        L = ora.Layer(top_k=TM.top_k(cfg), convention=ora.ATENIA, **TM.moe_arrays(t, layer))
        return L.block_forward(x1, gamma, eps, 0)[0]

    got, want = TM.logits(block, "deepseek_scale"), TM.hf_logits("deepseek_scale")
    assert 1e-3 < np.abs(got - want).max() < 1e-2
    assert np.array_equal(got.argmax(-1), want.argmax(-1))


def test_qwen_scale_detects_the_wrong_convention(ora):
    """Renormalised weights, an ungated shared expert or no shared expert at all each miss the
    HuggingFace logits by far more than the tolerance."""
    cfg, t = TM.load("qwen_scale")
    want = TM.hf_logits("qwen_scale")

    def with_(conv, drop_gate=False, drop_shared=False):
        def block(layer, x1, gamma, eps):
            a = TM.moe_arrays(t, layer)
            if drop_gate or drop_shared:
                a.pop("shared_gate")
            if drop_shared:
                for n in ("s_gate", "s_up", "s_down"):
                    a.pop(n)
            return ora.Layer(top_k=TM.top_k(cfg), convention=conv, **a).block_forward(x1, gamma, eps, 0)[0]
        return np.abs(TM.logits(block, "qwen_scale") - want).max()

    assert with_(ora.HUGGINGFACE_QWEN) < 1e-6
    assert with_(ora.ATENIA) > 1e-4                               # renormalised + ungated
    assert with_(ora.HUGGINGFACE_QWEN, drop_gate=True) > 1e-4     # raw weights, ungated shared
    assert with_(ora.HUGGINGFACE_QWEN, drop_shared=True) > 1e-4   # no shared expert


def test_tiny_mixtral_detects_a_broken_block(ora):
    """The fixture has teeth: no residual, no normalisation, or raw (not renormalised) top-k
    weights each move the logits far beyond the tolerance.  (Its gamma vectors are all ones, so
    gamma is pinned by the closed-form tests above, not here.)"""
    _, t = TM.load()

    def layer_of(i, conv=None):
        return ora.Layer(top_k=2, convention=ora.ATENIA if conv is None else conv, **TM.moe_arrays(t, i))

    def no_residual(layer, x1, gamma, eps):
        return layer_of(layer).block_forward(x1, gamma, eps, 0)[0] - x1

    def no_norm(layer, x1, gamma, eps):
        return x1 + layer_of(layer).execute(x1)[0]

    def no_renorm(layer, x1, gamma, eps):
        return layer_of(layer, ora.HUGGINGFACE_QWEN).block_forward(x1, gamma, eps, 0)[0]

    want = TM.hf_logits()
    for broken in (no_residual, no_norm, no_renorm):
        assert np.abs(TM.logits(broken) - want).max() > 1e-4, broken.__name__
