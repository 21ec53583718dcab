"""The decoder layer's FFN block on the GPU, out = x1 + MoE(RMSNorm(x1) * gamma), through the
C ABI (atenia_moe_hip_layer_block_forward[_device]) against the CPU oracle:

* the normalised rows (tap) are bit-identical to the oracle's under the f32 graph arithmetic --
  they feed the router, so routing stays bit-exact -- and within 1 ulp (almost all identical)
  under the f64 arithmetic, whose sum the kernel forms in a different order;
* the block equals residual + forward(normalised rows) bit for bit in every weight format;
* f32 layers meet the 1e-5 bar against the oracle's block, routing identical;
* the reference's whole-model fixture (HuggingFace f64 logits) with the GPU as every layer's block."""
import numpy as np
import pytest

from ateniaengine_amd import capi
from tests import synth as S
from tests import tiny_mixtral as TM
from tests.hipmem import DeviceArray

pytestmark = pytest.mark.gpu

EPS = 1e-5


def _rows(seed, T, d):
    """Residual-stream rows with the features that separate summation orders: wide spread of
    magnitudes inside a row, a head that swallows later squares in f32, an all-zero row."""
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((T, d)).astype(np.float32)
    x *= np.exp2(rng.integers(-6, 7, size=(T, d))).astype(np.float32)
    if T > 2:
        x[1] = 1.0
        x[1, 0] = 4096.0
        x[2] = 0.0
    return x


def _ulp(a, b):
    ia = np.ascontiguousarray(a, np.float32).view(np.int32).astype(np.int64)
    ib = np.ascontiguousarray(b, np.float32).view(np.int32).astype(np.int64)
    return np.abs(ia - ib)


@pytest.mark.parametrize("policy", [capi.NORM_GRAPH_F32, capi.NORM_F64])
@pytest.mark.parametrize("T,d,E,k,f", [(1, 4096, 8, 2, 64), (5, 50, 4, 2, 24), (16, 512, 8, 2, 32),
                                       (17, 1000, 6, 3, 40), (300, 256, 12, 3, 64)])
def test_block_f32_against_oracle(ora, policy, T, d, E, k, f):
    W = S.make_weights(d + T, E, d, f, router_std=1.0 / np.sqrt(d))
    oL, gL = S.build_pair(ora, W, k, capi.CONVENTION_ATENIA, capi.WEIGHT_F32)
    x1 = _rows(3 * T + d, T, d)
    gamma = (1.0 + 0.25 * np.random.default_rng(d).standard_normal(d)).astype(np.float32)
    with gL:
        out = gL.block_forward(x1, gamma, EPS, policy)
        h2 = gL.last_normed(T)
        idx = gL.last_routing(T)[0]
        o_out, o_h2, o_idx, _ = oL.block_forward(x1, gamma, EPS, policy)
        if policy == capi.NORM_GRAPH_F32:
            assert h2.tobytes() == o_h2.tobytes(), "normalised rows differ from the f32 graph arithmetic"
            assert np.array_equal(idx, o_idx)
        else:
            ul = _ulp(h2, o_h2)
            assert ul.max() <= 1 and (ul != 0).mean() <= 1e-4, (ul.max(), (ul != 0).mean())
            same = (ul.reshape(T, d) == 0).all(axis=1)
            assert np.array_equal(idx[same], o_idx[same])
        assert S.rel_err(out, o_out) <= 1e-5
        # composition: the block is the residual plus the op applied to the tap, bit for bit
        assert out.tobytes() == (x1 + gL.forward(h2).reshape(T, d)).astype(np.float32).tobytes()


@pytest.mark.parametrize("wd", [capi.WEIGHT_BF16, capi.WEIGHT_INT8_W8A16])
@pytest.mark.parametrize("T", [1, 16, 40, 600])
def test_block_throughput_formats_compose(ora, wd, T):
    d = 512
    W = S.make_weights(11, 8, d, 256, f_s=128, gated=True, router_std=1.0 / np.sqrt(d))
    oL, gL = S.build_pair(ora, W, 2, capi.CONVENTION_HUGGINGFACE_QWEN, wd)
    x1 = _rows(7 + T, T, d)
    gamma = (1.0 + 0.1 * np.random.default_rng(1).standard_normal(d)).astype(np.float32)
    with gL:
        out = gL.block_forward(x1, gamma, EPS, capi.NORM_GRAPH_F32)
        h2 = gL.last_normed(T)
        o_h2 = np.stack([ora.rms_norm_gamma(r, gamma, EPS, 0) for r in x1])
        assert h2.tobytes() == o_h2.tobytes()
        assert out.tobytes() == (x1 + gL.forward(h2).reshape(T, d)).astype(np.float32).tobytes()
        # and the layer output stays within the format's bar of the oracle on the stored weights
        ref = oL.block_forward(x1, gamma, EPS, 0)[0]
        assert S.rel_err(out - x1, ref - x1) <= 2e-2


def test_block_device_in_place(ora):
    T, d = 70, 256
    W = S.make_weights(5, 8, d, 128)
    _, gL = S.build_pair(ora, W, 2, capi.CONVENTION_ATENIA, capi.WEIGHT_BF16)
    x1 = _rows(1, T, d)
    gamma = np.linspace(0.5, 1.5, d).astype(np.float32)
    with gL:
        want = gL.block_forward(x1, gamma, EPS, capi.NORM_GRAPH_F32)
        dx, dg = DeviceArray.from_host(x1), DeviceArray.from_host(gamma)
        dout = DeviceArray((T, d), np.float32, fill=0)
        gL.block_forward_device(dx.ptr, T, dg.ptr, EPS, capi.NORM_GRAPH_F32, dout.ptr)
        assert gL.status()[0] == 0
        assert dout.to_host().tobytes() == want.tobytes()
        gL.block_forward_device(dx.ptr, T, dg.ptr, EPS, capi.NORM_GRAPH_F32, dx.ptr)  # in place
        assert gL.status()[0] == 0
        assert dx.to_host().tobytes() == want.tobytes()


def test_block_argument_errors(ora):
    W = S.make_weights(5, 4, 64, 32)
    _, gL = S.build_pair(ora, W, 2, capi.CONVENTION_ATENIA, capi.WEIGHT_F32)
    x1, g = np.ones((2, 64), np.float32), np.ones(64, np.float32)
    with gL:
        with pytest.raises(capi.MoeHipError) as e:
            gL.block_forward(x1, g, EPS, 7)
        assert e.value.rc == -1
        with pytest.raises(capi.MoeHipError) as e:
            gL.block_forward(x1, g, float("nan"), 0)
        assert e.value.rc == -1
        assert capi.lib().atenia_moe_hip_layer_last_normed(gL._h, None) == -1
        bad = x1.copy()
        bad[1, 3] = np.inf  # a non-finite row reaches the router as NaN and is reported, not hidden
        with pytest.raises(capi.MoeHipError) as e:
            gL.block_forward(bad, g, EPS, 0)
        assert e.value.rc == -3 and gL.last_non_finite()[0] == 1
        assert np.isfinite(gL.block_forward(x1, g, EPS, 0)).all()


@pytest.mark.parametrize("policy", [capi.NORM_GRAPH_F32, capi.NORM_F64])
def test_tiny_mixtral_logits_with_gpu_blocks(ora, policy):
    _, t = TM.load()
    layers = {}

    def block(layer, x1, gamma, eps):
        if layer not in layers:
            layers[layer] = capi.Layer(top_k=2, convention=capi.CONVENTION_ATENIA,
                                       weight_dtype=capi.WEIGHT_F32, **TM.moe_arrays(t, layer))
        return layers[layer].block_forward(x1, gamma, eps, policy)

    try:
        got, want = TM.logits(block), TM.hf_logits()
    finally:
        for L in layers.values():
            L.close()
    assert np.abs(got - want).max() < 1e-6
    assert np.array_equal(got.argmax(-1), want.argmax(-1))


@pytest.mark.parametrize("name,conv", [("mixtral_scale", capi.CONVENTION_ATENIA),
                                       ("qwen_scale", capi.CONVENTION_HUGGINGFACE_QWEN),
                                       ("deepseek_scale", capi.CONVENTION_HUGGINGFACE_QWEN)])
@pytest.mark.parametrize("policy", [capi.NORM_GRAPH_F32, capi.NORM_F64])
def test_scale_fixture_logits_with_gpu_blocks(ora, name, conv, policy):
    """The reference's topology fixtures (tests/moe_scale_cert_test.rs) with the GPU as every
    layer's FFN block: grouped-head Mixtral, Qwen2-MoE with its sigmoid-gated shared expert, and
    DeepSeek-V2 (top-6 of 16, two fused shared experts, latent attention in the NumPy part)."""
    cfg, t = TM.load(name)
    layers = {}

    def block(layer, x1, gamma, eps):
        if layer not in layers:
            layers[layer] = capi.Layer(top_k=TM.top_k(cfg), convention=conv,
                                       weight_dtype=capi.WEIGHT_F32, **TM.moe_arrays(t, layer))
        return layers[layer].block_forward(x1, gamma, eps, policy)

    try:
        got, want = TM.logits(block, name), TM.hf_logits(name)
    finally:
        for L in layers.values():
            L.close()
    assert np.abs(got - want).max() < 1e-6, np.abs(got - want).max()
    assert np.array_equal(got.argmax(-1), want.argmax(-1))
