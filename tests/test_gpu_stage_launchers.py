"""The four stage launchers (device pointers in, int code out) against the whole-pipeline entry
points: router -> permute -> expert_ffn -> combine, called one by one through the C ABI, must
reproduce atenia_moe_hip_layer_forward_device bit for bit, their routing / grouping taps must
equal the host-buffer taps (which the other tests hold against the CPU oracle), and a stage
called out of order must be refused."""
import numpy as np
import pytest

from ateniaengine_amd import capi
from tests import synth as S

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
    import torch

    oL, gL = _layer(ora, wd, gated)
    with gL:
        E, k, d = oL.E, oL.top_k, oL.d
        x = S.make_tokens(500 + T, T, d, bf16=wd != capi.WEIGHT_F32)
        dx = torch.from_numpy(x).cuda()
        whole = torch.empty((T, d), dtype=torch.float32, device="cuda")
        gL.forward_device(dx.data_ptr(), capi.ACT_F32, T, whole.data_ptr())
        torch.cuda.synchronize()
        assert gL.status()[0] == 0

        idx = torch.empty((T, k), dtype=torch.int32, device="cuda")
        w = torch.empty((T, k), dtype=torch.float32, device="cuda")
        counts = torch.empty((E,), dtype=torch.int32, device="cuda")
        offsets = torch.empty((E + 1,), dtype=torch.int32, device="cuda")
        perm = torch.empty((T * k,), dtype=torch.int32, device="cuda")
        staged = torch.zeros((T, d), dtype=torch.float32, device="cuda")
        gL.router_device(dx.data_ptr(), capi.ACT_F32, T, idx.data_ptr(), w.data_ptr())
        gL.permute_device(T, counts.data_ptr(), offsets.data_ptr(), perm.data_ptr())
        gL.expert_ffn_device(dx.data_ptr(), capi.ACT_F32, T)
        gL.combine_device(T, staged.data_ptr())
        torch.cuda.synchronize()
        assert torch.equal(staged, whole), "stages composed differ from the pipeline"

        h_idx, h_w = gL.route(x)
        assert np.array_equal(idx.cpu().numpy(), h_idx)
        assert np.array_equal(w.cpu().numpy().view(np.int32), h_w.view(np.int32))
        oc, oo, op = ora.permute(h_idx, E)
        assert np.array_equal(counts.cpu().numpy(), oc)
        assert np.array_equal(offsets.cpu().numpy(), oo)
        assert np.array_equal(perm.cpu().numpy(), op)


def test_stage_order_is_enforced(ora):
    import torch

    oL, gL = _layer(ora, capi.WEIGHT_BF16, False)
    with gL:
        T, d = 5, oL.d
        x = torch.from_numpy(S.make_tokens(9, T, d, bf16=True)).cuda()
        out = torch.empty((T, d), dtype=torch.float32, device="cuda")
        with pytest.raises(capi.MoeHipError) as e:
            gL.combine_device(T, out.data_ptr())
        assert e.value.rc == -1
        gL.router_device(x.data_ptr(), capi.ACT_F32, T)
        with pytest.raises(capi.MoeHipError):
            gL.expert_ffn_device(x.data_ptr(), capi.ACT_F32, T)  # permute has not run
        gL.permute_device(T)
        with pytest.raises(capi.MoeHipError):
            gL.combine_device(T + 1, out.data_ptr())  # other token count
        gL.expert_ffn_device(x.data_ptr(), capi.ACT_F32, T)
        gL.combine_device(T, out.data_ptr())
        torch.cuda.synchronize()
        assert torch.isfinite(out).all()
