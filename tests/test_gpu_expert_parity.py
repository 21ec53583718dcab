"""Per-expert parity at the benchmark shapes, exhaustive over experts.

The reference certifies a mixture-of-experts model expert by expert before it looks at the
combined output (docs/decisions/ADR-007-moe-certification-ladder.md:62-73, obligation C1:
"exhaustive (all experts), not sampled"; the generator computes h = silu(g@x)*(u@x); y = d@h one
expert at a time, fixtures/moe/generate_qwen_moe_decomposition_reference.py text lines 101-123),
and reports the routing margin next to the top-k set equality (ADR-007:75-88,
tests/moe_cert2_qwen_decomposition_test.rs:79-86).

Here, per benchmark configuration: a probe batch is built so that EVERY expert is selected at
least once (one engineered token per expert, pushed along that expert's router row, plus random
tokens so that the batch takes the kernel family of that size), the layer is forwarded through the
C ABI, and every tapped (token, slot) row of un-combined expert output -- and every row of the
shared expert's -- is compared with the oracle's all-f64 expert (`expert_forward_f64`) on the
stored weight values.  Bar: max|y - ref| / max|ref| per row <= 1e-2 (bf16 / int8) or 1e-5 (f32).
Routing is compared bit for bit first; the smallest routing margin of the batch is printed.
"""
import numpy as np
import pytest

from ateniaengine_amd import capi
from tests import synth as S

pytestmark = pytest.mark.gpu


def _normal(rng, shape, std):
    a = rng.standard_normal(shape, dtype=np.float32)
    a *= np.float32(std)
    return a


def probe_batch(rng, w_router, T, bf16, lift=9.0):
    """T tokens ~ N(0, 1); token e (e < E) is moved along router row e so that expert e's logit
    rises by `lift` logit standard deviations and the token selects it."""
    E, d = w_router.shape
    x = rng.standard_normal((T, d), dtype=np.float32)
    for e in range(min(E, T)):
        r = w_router[e].astype(np.float64)
        sd = np.sqrt((r * r).sum())  # std of a logit under x ~ N(0, 1)
        x[e] += (lift * r / sd).astype(np.float32)
    return S.bf16_round_trip(x)[1] if bf16 else x


def check_every_expert(ora, oL, gL, x, tol, label, expect_family=None):
    T = x.shape[0]
    if expect_family is not None:
        assert gL.expert_kernels(T)[0] == expect_family, (label, gL.expert_kernels(T))
    gL.forward(x)
    idx, w, counts, _, _ = gL.last_routing(T)
    o_idx, _, logits = oL.route_tokens(x, want_logits=True)
    assert (idx == o_idx).all(), f"{label}: routing differs from the CPU path"
    assert (counts > 0).all(), f"{label}: experts without a token: {np.nonzero(counts == 0)[0]}"
    srt = np.sort(logits.astype(np.float64), axis=1)[:, ::-1]
    margin = float((srt[:, oL.top_k - 1] - srt[:, oL.top_k]).min())
    y, ys = gL.last_expert_outputs(T)
    worst, worst_at = 0.0, None
    per_expert = np.zeros(oL.E)
    for t in range(T):
        for s, e in enumerate(idx[t]):
            ref = ora.expert_forward_f64(oL.w_gate[e], oL.w_up[e], oL.w_down[e], x[t])
            err = S.rel_err(y[t, s], ref)
            per_expert[e] = max(per_expert[e], err)
            if err > worst:
                worst, worst_at = err, (t, s, int(e))
    assert worst <= tol, f"{label}: expert output off by {worst:.3e} at (token, slot, expert) {worst_at}"
    worst_s = 0.0
    if oL.f_s:
        for t in range(T):
            ref = ora.expert_forward_f64(oL.s_gate, oL.s_up, oL.s_down, x[t])
            worst_s = max(worst_s, S.rel_err(ys[t], ref))
        assert worst_s <= tol, f"{label}: shared expert output off by {worst_s:.3e}"
    print(f"{label}: T={T}, {T * oL.top_k} expert rows over all {oL.E} experts, worst {worst:.2e} "
          f"(best-covered expert {per_expert.min():.1e}), shared {worst_s:.2e}, min routing margin "
          f"{margin:.3e}")


@pytest.fixture(scope="module")
def threads(ora):
    ora.set_threads(ora.hw_threads())
    yield
    ora.set_threads(1)


def test_config1_tiny_f32_every_expert(ora, threads):
    rng = np.random.default_rng(111)
    E, k, d, f = 8, 2, 1024, 2048
    W = dict(w_router=_normal(rng, (E, d), 0.02), w_gate=_normal(rng, (E, f, d), 0.02),
             w_up=_normal(rng, (E, f, d), 0.02), w_down=_normal(rng, (E, d, f), 0.02))
    oL, gL = S.build_pair(ora, W, k, capi.CONVENTION_ATENIA, capi.WEIGHT_F32)
    with gL:
        x = probe_batch(rng, oL.w_router, 64, bf16=False)
        check_every_expert(ora, oL, gL, x, 1e-5, "config1 f32")


@pytest.fixture(scope="module")
def mixtral_weights():
    rng = np.random.default_rng(212)
    E, d, f = 8, 4096, 14336
    return dict(w_router=_normal(rng, (E, d), 0.02), w_gate=_normal(rng, (E, f, d), 0.02),
                w_up=_normal(rng, (E, f, d), 0.02), w_down=_normal(rng, (E, d, f), 0.02))


def test_config2_mixtral_bf16_every_expert(ora, threads, mixtral_weights):
    oL, gL = S.build_pair(ora, mixtral_weights, 2, capi.CONVENTION_ATENIA, capi.WEIGHT_BF16,
                          max_tokens_hint=320)
    rng = np.random.default_rng(213)
    with gL:
        # decode kernels (16 tokens) and the matrix-core tiled kernels (320 tokens = 80 rows per expert)
        check_every_expert(ora, oL, gL, probe_batch(rng, oL.w_router, 16, True), 1e-2,
                           "config2 mixtral bf16 (streaming)", capi.KERNELS_STREAM)
        check_every_expert(ora, oL, gL, probe_batch(rng, oL.w_router, 320, True), 1e-2,
                           "config2 mixtral bf16 (tiled)", capi.KERNELS_TILED)
    del oL


def test_config3_mixtral_int8_every_expert(ora, threads, mixtral_weights):
    W = dict(mixtral_weights)
    rng = np.random.default_rng(313)
    for name in ("w_gate", "w_up", "w_down"):  # 0.1 % of output channels carry x8 magnitude
        a = W[name] = W[name].copy()
        rows = a.reshape(-1, a.shape[-1])
        rows[rng.choice(rows.shape[0], size=rows.shape[0] // 1000, replace=False)] *= 8.0
    oL, gL = S.build_pair(ora, W, 2, capi.CONVENTION_ATENIA, capi.WEIGHT_INT8_W8A16,
                          max_tokens_hint=448)
    del W
    with gL:
        check_every_expert(ora, oL, gL, probe_batch(rng, oL.w_router, 16, True), 1e-2,
                           "config3 mixtral int8 (streaming)", capi.KERNELS_STREAM)
        check_every_expert(ora, oL, gL, probe_batch(rng, oL.w_router, 448, True), 1e-2,
                           "config3 mixtral int8 (tiled)", capi.KERNELS_TILED)
    del oL


def test_config4_qwen_bf16_every_expert(ora, threads):
    rng = np.random.default_rng(414)
    E, k, d, f, fs = 60, 4, 2048, 1408, 5632
    W = dict(w_router=_normal(rng, (E, d), 1.0 / np.sqrt(d)), w_gate=_normal(rng, (E, f, d), 0.02),
             w_up=_normal(rng, (E, f, d), 0.02), w_down=_normal(rng, (E, d, f), 0.02),
             s_gate=_normal(rng, (fs, d), 0.02), s_up=_normal(rng, (fs, d), 0.02),
             s_down=_normal(rng, (d, fs), 0.02), shared_gate=_normal(rng, (d,), 0.02))
    oL, gL = S.build_pair(ora, W, k, capi.CONVENTION_HUGGINGFACE_QWEN, capi.WEIGHT_BF16,
                          max_tokens_hint=2048)
    del W
    with gL:
        check_every_expert(ora, oL, gL, probe_batch(rng, oL.w_router, 96, True), 1e-2,
                           "config4 qwen bf16 (mid-batch)", capi.KERNELS_MID)
        check_every_expert(ora, oL, gL, probe_batch(rng, oL.w_router, 2048, True), 1e-2,
                           "config4 qwen bf16 (tiled)", capi.KERNELS_TILED)


def test_config5_deepseek_bf16_every_expert(ora, threads):
    rng = np.random.default_rng(515)
    E, k, d, f, fs = 64, 6, 2048, 1408, 2816
    bias = (-1.2 * np.log(rng.permutation(E) + 1.0)).astype(np.float32)  # log-Zipf(1.2)
    W = dict(w_router=_normal(rng, (E, d), 1.0 / np.sqrt(d)), w_gate=_normal(rng, (E, f, d), 0.02),
             w_up=_normal(rng, (E, f, d), 0.02), w_down=_normal(rng, (E, d, f), 0.02),
             s_gate=_normal(rng, (fs, d), 0.02), s_up=_normal(rng, (fs, d), 0.02),
             s_down=_normal(rng, (d, fs), 0.02), router_bias=bias)
    oL, gL = S.build_pair(ora, W, k, capi.CONVENTION_HUGGINGFACE_QWEN, capi.WEIGHT_BF16,
                          max_tokens_hint=1536)
    del W
    with gL:
        # the least likely expert (bias -1.2 ln 64 = -5) is reached only by its engineered token
        check_every_expert(ora, oL, gL, probe_batch(rng, oL.w_router, 64, True, lift=12.0), 1e-2,
                           "config5 deepseek bf16 (mid-batch)", capi.KERNELS_MID)
        check_every_expert(ora, oL, gL, probe_batch(rng, oL.w_router, 1536, True, lift=12.0), 1e-2,
                           "config5 deepseek bf16 (tiled)", capi.KERNELS_TILED)
