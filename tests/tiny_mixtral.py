"""The whole-model fixtures `full_mixtral` (2 layers, hidden 32, 4 heads, 4 experts, top-2, 5
tokens), `mixtral_scale` (hidden 64, 8 heads over 2 key/value heads, 8 experts, top-2) and
`qwen_scale` (16 experts, top-4 without renormalisation, sigmoid-gated shared expert, grouped
heads with q/k/v bias) and `deepseek_scale` (16 experts, top-6 renormalised, two fused ungated
shared experts, multi-head latent attention) -- weights + HuggingFace f64 logits --, used to pin the decoder-layer FFN block
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
SCALE = ("mixtral_scale", "qwen_scale", "deepseek_scale")


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
    if p + "shared_experts.gate_proj.weight" in t:  # DeepSeek: fused shared experts, no gate
        a.update(s_gate=t[p + "shared_experts.gate_proj.weight"], s_up=t[p + "shared_experts.up_proj.weight"],
                 s_down=t[p + "shared_experts.down_proj.weight"])
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


def _attention_mla(h, t, p, cfg):
    """DeepSeek-V2 multi-head latent attention as src/moe/mla.rs:300-420 runs it: low-rank
    key/value compression with its own RMSNorm, a no-rope and a rope part per head, the key's
    rope part shared by all heads, interleaved rotary pairs (2i, 2i+1), scale qk_head_dim^-0.5."""
    seq, nh = h.shape[0], cfg["num_attention_heads"]
    nope, rope, vd, kvl = (cfg[k] for k in ("qk_nope_head_dim", "qk_rope_head_dim", "v_head_dim",
                                            "kv_lora_rank"))
    w = lambda n: t[p + f"self_attn.{n}.weight"].astype(np.float64)
    q = (h @ w("q_proj").T).reshape(seq, nh, nope + rope)
    ckv = h @ w("kv_a_proj_with_mqa").T
    # HuggingFace builds kv_a_layernorm with its class default eps = 1e-6, not the config's
    # rms_norm_eps (with the config's 1e-5 the logits are 4.8e-5 off, with 1e-6 they match to 5e-8)
    kv = (_rms(ckv[:, :kvl], t[p + "self_attn.kv_a_layernorm.weight"], 1e-6)
          @ w("kv_b_proj").T).reshape(seq, nh, nope + vd)
    inv_freq = 1.0 / cfg["rope_theta"] ** (np.arange(0, rope, 2, dtype=np.float64) / rope)
    ang = np.arange(seq, dtype=np.float64)[:, None] * inv_freq[None, :]

    def rot(x):  # x [..., rope] with positions along axis 0
        a, b = x[..., 0::2], x[..., 1::2]
        c, s_ = np.cos(ang), np.sin(ang)
        while c.ndim < a.ndim:
            c, s_ = c[:, None], s_[:, None]
        out = np.empty_like(x)
        out[..., 0::2], out[..., 1::2] = a * c - b * s_, a * s_ + b * c
        return out

    qh = np.concatenate([q[..., :nope], rot(q[..., nope:])], -1).transpose(1, 0, 2)
    k_pe = np.broadcast_to(rot(ckv[:, kvl:])[:, None, :], (seq, nh, rope))
    kh = np.concatenate([kv[..., :nope], k_pe], -1).transpose(1, 0, 2)
    vh = kv[..., nope:].transpose(1, 0, 2)
    s = qh @ kh.transpose(0, 2, 1) / np.sqrt(nope + rope)
    s = np.where(np.tril(np.ones((seq, seq), bool)), s, -np.inf)
    s = np.exp(s - s.max(-1, keepdims=True))
    a = s / s.sum(-1, keepdims=True)
    return (a @ vh).transpose(1, 0, 2).reshape(seq, nh * vd) @ w("o_proj").T


def logits(block_fn, name=NAME):
    """Logits [seq, vocab] with `block_fn(layer, x1_f32[seq, hidden], gamma_f32, eps) -> f32
    [seq, hidden]` as every layer's FFN block."""
    cfg, t = load(name)
    eps = cfg["rms_norm_eps"]
    x = t["model.embed_tokens.weight"][np.array(cfg["input_ids"])].astype(np.float64)
    for layer in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{layer}."
        attend = _attention_mla if cfg.get("model_type") == "deepseek_v2" else _attention
        x1 = x + attend(_rms(x, t[p + "input_layernorm.weight"], eps), t, p, cfg)
        x1 = x1.astype(np.float32)  # the residual stream is f32 where the block takes over
        x = np.asarray(block_fn(layer, x1, t[p + "post_attention_layernorm.weight"], eps),
                       dtype=np.float64).reshape(x1.shape)
    return _rms(x, t["model.norm.weight"], eps) @ t["lm_head.weight"].astype(np.float64).T


def hf_logits(name=NAME):
    cfg, _ = load(name)
    return np.array(cfg["hf_logits"], dtype=np.float64).reshape(cfg["seq"], cfg["vocab_size"])
