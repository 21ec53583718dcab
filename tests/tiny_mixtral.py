"""The whole-model fixtures `full_mixtral` (2 layers, hidden 32, 4 heads, 4 experts, top-2, 5
tokens), `mixtral_scale` (hidden 64, 8 heads over 2 key/value heads, 8 experts, top-2) and
`qwen_scale` (16 experts, top-4 without renormalisation, sigmoid-gated shared expert, grouped
heads with q/k/v bias) -- weights + HuggingFace f64 logits --, used to pin the decoder-layer FFN block
`x1 + MoE(RMSNorm(x1) * gamma)` from outside: everything except that block is computed here in
NumPy f64 (embedding, input norm, rotary attention, final norm, lm_head -- the standard
Mixtral layer as the reference's tests/moe_full_forward_test.rs:140-165 runs it), the block is
supplied by the caller (the CPU oracle or the GPU path).  A missing residual, a norm without
the mean or a wrong routing convention in the block moves the logits by far more than the
tolerance.  The fixture's norm weights are all ones (a freshly initialised model), so gamma is
pinned by closed-form tests instead."""
import json
import os

import numpy as np

from tests import golden_io as G

NAME = "full_mixtral"
SCALE = ("mixtral_scale", "qwen_scale")


def load(name=NAME):
    """(config + sidecar as one dict, tensors)."""
    cfg = dict(G.sidecar(name))
    extra = os.path.join(G.GOLDEN, name + "_config.json")
    if os.path.exists(extra):
        with open(extra) as fp:
            cfg.update(json.load(fp))
    cfg.setdefault("head_dim", cfg["hidden_size"] // cfg["num_attention_heads"])
    return cfg, G.tensors(name)


def top_k(cfg):
    return int(cfg["num_experts_per_tok"])


def moe_arrays(t, layer):
    """Arrays of layer `layer`'s MoE block in the form oracle.Layer / capi.Layer take."""
    p = f"model.layers.{layer}.mlp."
    gu = t[p + "experts.gate_up_proj"]
    f = gu.shape[1] // 2
    a = dict(w_router=t[p + "gate.weight"], w_gate=np.ascontiguousarray(gu[:, :f, :]),
             w_up=np.ascontiguousarray(gu[:, f:, :]), w_down=t[p + "experts.down_proj"])
    if p + "shared_expert.gate_proj.weight" in t:
        a.update(s_gate=t[p + "shared_expert.gate_proj.weight"], s_up=t[p + "shared_expert.up_proj.weight"],
                 s_down=t[p + "shared_expert.down_proj.weight"],
                 shared_gate=np.ascontiguousarray(t[p + "shared_expert_gate.weight"].reshape(-1)))
    return a


def _rms(x, g, eps):
    x = x.astype(np.float64)
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps) * g.astype(np.float64)


def _rotate_half(x):
    h = x.shape[-1] // 2
    return np.concatenate([-x[..., h:], x[..., :h]], axis=-1)


def _attention(h, t, p, cfg):
    seq, nh, hd = h.shape[0], cfg["num_attention_heads"], cfg["head_dim"]
    nkv = cfg.get("num_key_value_heads", nh)

    def proj(n):
        y = h @ t[p + f"self_attn.{n}_proj.weight"].astype(np.float64).T
        b = t.get(p + f"self_attn.{n}_proj.bias")
        return y if b is None else y + b.astype(np.float64)

    q = proj("q").reshape(seq, nh, hd).transpose(1, 0, 2)
    k, v = (proj(n).reshape(seq, nkv, hd).transpose(1, 0, 2) for n in "kv")
    k, v = (np.repeat(a, nh // nkv, axis=0) for a in (k, v))  # grouped heads share k / v
    inv_freq = 1.0 / cfg["rope_theta"] ** (np.arange(0, hd, 2, dtype=np.float64) / hd)
    ang = np.arange(seq, dtype=np.float64)[:, None] * inv_freq[None, :]
    cos, sin = (np.concatenate([fn(ang), fn(ang)], -1) for fn in (np.cos, np.sin))
    q = q * cos + _rotate_half(q) * sin
    k = k * cos + _rotate_half(k) * sin
    s = q @ k.transpose(0, 2, 1) / np.sqrt(hd)
    s = np.where(np.tril(np.ones((seq, seq), bool)), s, -np.inf)
    s = np.exp(s - s.max(-1, keepdims=True))
    a = s / s.sum(-1, keepdims=True)
    ctx = (a @ v).transpose(1, 0, 2).reshape(seq, nh * hd)
    return ctx @ t[p + "self_attn.o_proj.weight"].astype(np.float64).T


def logits(block_fn, name=NAME):
    """Logits [seq, vocab] with `block_fn(layer, x1_f32[seq, hidden], gamma_f32, eps) -> f32
    [seq, hidden]` as every layer's FFN block."""
    cfg, t = load(name)
    eps = cfg["rms_norm_eps"]
    x = t["model.embed_tokens.weight"][np.array(cfg["input_ids"])].astype(np.float64)
    for layer in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{layer}."
        x1 = x + _attention(_rms(x, t[p + "input_layernorm.weight"], eps), t, p, cfg)
        x1 = x1.astype(np.float32)  # the residual stream is f32 where the block takes over
        x = np.asarray(block_fn(layer, x1, t[p + "post_attention_layernorm.weight"], eps),
                       dtype=np.float64).reshape(x1.shape)
    return _rms(x, t["model.norm.weight"], eps) @ t["lm_head.weight"].astype(np.float64).T


def hf_logits(name=NAME):
    cfg, _ = load(name)
    return np.array(cfg["hf_logits"], dtype=np.float64).reshape(cfg["seq"], cfg["vocab_size"])
