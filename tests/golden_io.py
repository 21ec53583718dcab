"""Loads the golden fixtures under tests/golden into oracle.Layer objects."""
import json
import os

import numpy as np
from safetensors.numpy import load_file

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")

LAYER0 = ["mixtral_layer0", "qwen15_moe_layer0", "qwen2_moe_layer0", "qwen3_moe_layer0"]


def sidecar(name):
    with open(os.path.join(GOLDEN, name + ".json")) as f:
        return json.load(f)


def tensors(name):
    return load_file(os.path.join(GOLDEN, name + ".safetensors"))


def _find(t, suffixes):
    for k in t:
        for s in suffixes:
            if k.endswith(s):
                return t[k]
    return None


def layer_arrays(name):
    """dict of f32 arrays: router [E,d], gate/up [E,f,d], down [E,d,f], shared*, shared_gate.

    Packed experts are `[E, 2f, d]` with gate = rows 0..f, up = rows f..2f
    (reference src/moe/binding.rs:384-413)."""
    t = tensors(name)
    gu = _find(t, [".experts.gate_up_proj"])
    f = gu.shape[1] // 2
    out = dict(
        w_router=_find(t, [".gate.weight", ".router.weight"]),
        w_gate=np.ascontiguousarray(gu[:, :f, :]),
        w_up=np.ascontiguousarray(gu[:, f:, :]),
        w_down=_find(t, [".experts.down_proj"]),
        s_gate=_find(t, ["shared_expert.gate_proj.weight", "shared_experts.gate_proj.weight"]),
        s_up=_find(t, ["shared_expert.up_proj.weight", "shared_experts.up_proj.weight"]),
        s_down=_find(t, ["shared_expert.down_proj.weight", "shared_experts.down_proj.weight"]),
        shared_gate=_find(t, ["shared_expert_gate.weight"]),
    )
    if out["shared_gate"] is not None:
        out["shared_gate"] = out["shared_gate"].reshape(-1)
    return out


def oracle_layer(ora, name, top_k, convention):
    a = layer_arrays(name)
    return ora.Layer(top_k=top_k, convention=convention, **a)


def v3_arrays():
    """The DeepSeek-V3 routing fixture as layer arrays (8 experts, one shared expert)."""
    t = tensors("v3_route_ref")
    n = sidecar("v3_route_ref")["n_routed_experts"]
    st = lambda part: np.stack([t[f"expert.{e}.{part}"] for e in range(n)])
    return dict(w_router=t["router.weight"], w_gate=st("w_gate"), w_up=st("w_up"), w_down=st("w_down"),
                s_gate=t["shared.w_gate"], s_up=t["shared.w_up"], s_down=t["shared.w_down"])


def v3_oracle_layer(ora):
    return ora.Layer(top_k=sidecar("v3_route_ref")["top_k"], convention=ora.HUGGINGFACE_QWEN,
                     **v3_arrays())
