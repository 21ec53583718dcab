"""Pins the `router_bias` term of the oracle's router independently of the oracle's own code.

The reference router has NO bias term (src/moe/dense.rs:325-337: route = matvec + softmax), so
no reference fixture can hold this arithmetic.  The benchmark's skewed-load configuration adds a
per-expert bias to the f32 logits before the softmax; what that has to mean is fixed here from
pieces that ARE pinned elsewhere:

  logit[e] = (f32) sum_c (f64)w[e,c] * (f64)x[c]        c ascending   (dense.rs:97-115, KATs in
                                                                        test_oracle_kat.py)
  logit[e] = logit[e] + bias[e]                          one f32 addition
  weights  = softmax(logits)                              (dense.rs:172-187, pinned by KATs)
  routing  = top_k_routing_with(weights, k, renorm)       (sparse.rs:142-191, pinned by KATs)

The dot product below is NumPy (f64 cumulative sum = the sequential order), not the oracle's
matvec; softmax and top-k are the oracle's pinned functions applied to logits this file forms.
A bias added in f64 before the rounding, a bias subtracted, a bias added after the softmax or a
bias indexed by slot instead of expert all fail at least one case here.
"""
import numpy as np
import pytest


def np_logits(w_router, x, bias):
    """[T, E] f32 logits: sequential f64 dot, rounded to f32, then one f32 add of the bias."""
    prod = w_router.astype(np.float64)[None, :, :] * x.astype(np.float64)[:, None, :]
    dots = np.cumsum(prod, axis=2)[:, :, -1]  # cumsum adds left to right
    lo = dots.astype(np.float32)
    return (lo + bias.astype(np.float32)[None, :]).astype(np.float32)


def route_from_logits(ora, logits, k, renorm):
    T = logits.shape[0]
    idx = np.empty((T, k), dtype=np.int32)
    w = np.empty((T, k), dtype=np.float32)
    for t in range(T):
        idx[t], w[t] = ora.top_k_routing_with(ora.softmax(logits[t]), k, renormalize=renorm)
    return idx, w


def zipf_bias(E, seed):
    rank = np.random.default_rng(seed).permutation(E) + 1.0
    return (-1.2 * np.log(rank)).astype(np.float32)


def layer_with_bias(ora, w_router, bias, k, conv):
    E, d = w_router.shape
    z = np.zeros((E, 1, d), dtype=np.float32)
    return ora.Layer(w_router=w_router, w_gate=z, w_up=z, w_down=np.zeros((E, d, 1), np.float32),
                     top_k=k, convention=conv, router_bias=bias)


@pytest.mark.parametrize("E,k,d,conv", [(8, 2, 64, 0), (64, 6, 48, 1), (60, 4, 32, 1)])
def test_route_with_bias_equals_independent_restatement(ora, E, k, d, conv):
    rng = np.random.default_rng(100 + E)
    w_router = (rng.standard_normal((E, d)) / np.sqrt(d)).astype(np.float32)
    x = rng.standard_normal((1200, d)).astype(np.float32)
    bias = zipf_bias(E, 7)
    L = layer_with_bias(ora, w_router, bias, k, conv)
    idx, w, lo = L.route_tokens(x, want_logits=True)
    ref_lo = np_logits(w_router, x, bias)
    assert (lo.view(np.uint32) == ref_lo.view(np.uint32)).all()
    ref_idx, ref_w = route_from_logits(ora, ref_lo, k, conv == 0)
    assert (idx == ref_idx).all()
    assert (w.view(np.uint32) == ref_w.view(np.uint32)).all()


def test_bias_is_added_in_f32_after_the_rounding(ora):
    """f32(dot) + bias in f32 differs from f32(dot + bias) on enough logits that the test
    inputs tell the two apart; the oracle must follow the first."""
    rng = np.random.default_rng(5)
    E, d = 16, 40
    w_router = rng.standard_normal((E, d)).astype(np.float32)
    x = rng.standard_normal((400, d)).astype(np.float32)
    bias = zipf_bias(E, 3)
    L = layer_with_bias(ora, w_router, bias, 2, 0)
    _, _, lo = L.route_tokens(x, want_logits=True)
    prod = w_router.astype(np.float64)[None] * x.astype(np.float64)[:, None, :]
    dots = np.cumsum(prod, axis=2)[:, :, -1]
    wrong = (dots + bias.astype(np.float64)[None]).astype(np.float32)
    right = np_logits(w_router, x, bias)
    assert (wrong.view(np.uint32) != right.view(np.uint32)).any(), "inputs do not separate the forms"
    assert (lo.view(np.uint32) == right.view(np.uint32)).all()


def test_zero_router_reduces_to_softmax_of_the_bias(ora):
    """W_r = 0 makes every logit exactly its bias: the weights are the closed-form softmax of
    the bias vector (computed here in plain f64) and the top-k are its k largest entries."""
    E, d, k = 10, 16, 3
    bias = np.array([0.5, -1.0, 2.0, 0.0, 1.5, -0.25, 2.0, 0.75, -3.0, 1.0], dtype=np.float32)
    L = layer_with_bias(ora, np.zeros((E, d), np.float32), bias, k, 1)
    x = np.random.default_rng(1).standard_normal((5, d)).astype(np.float32)
    idx, w, lo = L.route_tokens(x, want_logits=True)
    assert (lo == bias[None]).all()
    e = np.exp(bias.astype(np.float64) - 2.0)
    closed = e / e.sum()
    # the two 2.0 entries tie: lower index first, then 1.5; emitted ascending
    assert (idx == np.array([2, 4, 6])).all()
    assert np.abs(w - closed[[2, 4, 6]].astype(np.float32)[None]).max() <= 1e-7


def test_bias_breaks_and_makes_ties(ora):
    """Exactly representable logits: a bias that lifts expert 3 onto expert 1's logit makes a tie
    that the lower index wins; a larger bias makes expert 3 win outright."""
    E, d = 4, 2
    w_router = np.array([[0.0, 0.0], [1.0, 0.0], [0.0, 0.0], [0.5, 0.0]], dtype=np.float32)
    x = np.array([[1.0, 0.0]], dtype=np.float32)
    for lift, want in ((np.float32(0.5), [1]), (np.float32(0.75), [3])):
        bias = np.array([0, 0, 0, lift], dtype=np.float32)
        idx, _ = layer_with_bias(ora, w_router, bias, 1, 1).route_tokens(x)
        assert idx.tolist() == [want]
    # a negative bias removes the otherwise best expert from the selection
    bias = np.array([0, -2, 0, 0], dtype=np.float32)
    idx, _ = layer_with_bias(ora, w_router, bias, 2, 1).route_tokens(x)
    assert idx.tolist() == [[0, 3]]


def test_bias_is_indexed_by_expert_and_absent_means_zero(ora):
    rng = np.random.default_rng(9)
    E, d, k = 12, 24, 3
    w_router = rng.standard_normal((E, d)).astype(np.float32)
    x = rng.standard_normal((50, d)).astype(np.float32)
    zero = layer_with_bias(ora, w_router, np.zeros(E, np.float32), k, 0).route_tokens(x)
    none = layer_with_bias(ora, w_router, None, k, 0).route_tokens(x)
    assert (zero[0] == none[0]).all() and (zero[1].view(np.uint32) == none[1].view(np.uint32)).all()
    # +40 on one expert puts it into every token's selection, and only that expert
    for e in (0, 5, 11):
        bias = np.zeros(E, np.float32)
        bias[e] = 40.0
        idx, _ = layer_with_bias(ora, w_router, bias, k, 0).route_tokens(x)
        assert (idx == e).any(axis=1).all()
