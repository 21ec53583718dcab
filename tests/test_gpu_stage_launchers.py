"""The four stage launchers (device pointers in, int code out) against the whole-pipeline entry
points: router -> permute -> expert_ffn -> combine, called one by one through the C ABI, must
reproduce atenia_moe_hip_layer_forward_device bit for bit, their routing / grouping taps must
equal the host-buffer taps (which the other tests hold against the CPU oracle), and a stage
called out of order must be refused."""
import numpy as np
import pytest

from ateniaengine_amd import capi
from tests import synth as S
from tests.hipmem import DeviceArray

pytestmark = pytest.mark.gpu


def _layer(ora, wd, gated):
    W = S.make_weights(77, 12, 256, 192, f_s=128 if gated else 0, gated=gated,
                       router_std=1.0 / 16.0)
    conv = capi.CONVENTION_HUGGINGFACE_QWEN if gated else capi.CONVENTION_ATENIA
    return S.build_pair(ora, W, 3, conv, wd)


@pytest.mark.parametrize("wd,gated", [(capi.WEIGHT_BF16, False), (capi.WEIGHT_BF16, True),
                                      (capi.WEIGHT_INT8_W8A16, False), (capi.WEIGHT_F32, True)])
@pytest.mark.parametrize("T", [1, 19, 300])
def test_stages_equal_pipeline(ora, wd, gated, T):
    oL, gL = _layer(ora, wd, gated)
    with gL:
        E, k, d = oL.E, oL.top_k, oL.d
        x = S.make_tokens(500 + T, T, d, bf16=wd != capi.WEIGHT_F32)
        dx = DeviceArray.from_host(x)
        whole = DeviceArray((T, d), np.float32, fill=0)
        gL.forward_device(dx.ptr, capi.ACT_F32, T, whole.ptr)
        assert gL.status()[0] == 0
        want = whole.to_host()

        idx = DeviceArray((T, k), np.int32)
        w = DeviceArray((T, k), np.float32)
        counts = DeviceArray((E,), np.int32)
        offsets = DeviceArray((E + 1,), np.int32)
        perm = DeviceArray((T * k,), np.int32)
        staged = DeviceArray((T, d), np.float32, fill=0)
        gL.router_device(dx.ptr, capi.ACT_F32, T, idx.ptr, w.ptr)
        gL.permute_device(T, counts.ptr, offsets.ptr, perm.ptr)
        gL.expert_ffn_device(dx.ptr, capi.ACT_F32, T)
        gL.combine_device(T, staged.ptr)
        assert staged.to_host().tobytes() == want.tobytes(), "stages composed differ from the pipeline"
        ref = oL.execute(x)[0] if wd == capi.WEIGHT_F32 else None
        if ref is not None:  # f32 layers: also against the certified CPU path itself
            assert S.rel_err(want, ref) <= 1e-5

        h_idx, h_w = gL.route(x)
        assert np.array_equal(idx.to_host(), h_idx)
        assert np.array_equal(w.to_host().view(np.int32), h_w.view(np.int32))
        oc, oo, op = ora.permute(h_idx, E)
        assert np.array_equal(counts.to_host(), oc)
        assert np.array_equal(offsets.to_host(), oo)
        assert np.array_equal(perm.to_host(), op)


def test_stage_order_is_enforced(ora):
    oL, gL = _layer(ora, capi.WEIGHT_BF16, False)
    with gL:
        T, d = 5, oL.d
        x = DeviceArray.from_host(S.make_tokens(9, T, d, bf16=True))
        out = DeviceArray((T + 1, d), np.float32, fill=0)
        with pytest.raises(capi.MoeHipError) as e:
            gL.combine_device(T, out.ptr)
        assert e.value.rc == -1
        gL.router_device(x.ptr, capi.ACT_F32, T)
        with pytest.raises(capi.MoeHipError):
            gL.expert_ffn_device(x.ptr, capi.ACT_F32, T)  # permute has not run
        gL.permute_device(T)
        with pytest.raises(capi.MoeHipError):
            gL.combine_device(T + 1, out.ptr)  # other token count
        gL.expert_ffn_device(x.ptr, capi.ACT_F32, T)
        gL.combine_device(T, out.ptr)
        assert np.isfinite(out.to_host()).all()


@pytest.mark.parametrize("wd", [capi.WEIGHT_BF16, capi.WEIGHT_INT8_W8A16])
@pytest.mark.parametrize("k", [1, 2])
def test_single_token_fused_down_and_combine(ora, wd, k):
    """One token with up to two experts per token: the pipeline's down launch also does the
    combine.  It must give the bits of the stages called one by one (which use the separate
    down and combine kernels), also with a residual (the block entry point), and leave the same
    per-expert outputs in the tap."""
    d = 512
    W = S.make_weights(300 + k, 8, d, 1024, router_std=1.0 / 16.0)
    oL, gL = S.build_pair(ora, W, k, capi.CONVENTION_ATENIA, wd)
    with gL:
        for seed in range(4):
            x = S.make_tokens(900 + seed, 1, d)
            dx = DeviceArray.from_host(x)
            whole = DeviceArray((1, d), np.float32, fill=0)
            gL.forward_device(dx.ptr, capi.ACT_F32, 1, whole.ptr)
            assert gL.status()[0] == 0
            y_fused = gL.last_expert_outputs(1)[0]
            assert gL.stage_launches()[4] == 0, "the combine launch must be gone"
            staged = DeviceArray((1, d), np.float32, fill=0)
            gL.router_device(dx.ptr, capi.ACT_F32, 1)
            gL.permute_device(1)
            gL.expert_ffn_device(dx.ptr, capi.ACT_F32, 1)
            gL.combine_device(1, staged.ptr)
            assert gL.stage_launches()[4] == 1
            assert whole.to_host().tobytes() == staged.to_host().tobytes()
            assert y_fused.tobytes() == gL.last_expert_outputs(1)[0].tobytes()
            assert S.rel_err(whole.to_host(), oL.execute(x)[0]) <= 2e-2
        x1 = S.make_tokens(77, 1, d, bf16=False)
        gamma = np.linspace(0.8, 1.2, d).astype(np.float32)
        blk = gL.block_forward(x1, gamma, 1e-5, capi.NORM_GRAPH_F32)
        h2 = gL.last_normed(1)
        assert blk.tobytes() == (x1 + gL.forward(h2).reshape(1, d)).astype(np.float32).tobytes()
