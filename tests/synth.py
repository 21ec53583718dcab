"""Synthetic layers shared by the parity tests: the same host arrays feed the CPU oracle and
the HIP library, so both see identical stored weight values."""
import numpy as np

from ateniaengine_amd import capi


def bf16_round_trip(a):
    """f32 -> bf16 (truncation, reference src/tensor/tensor.rs:306-308) -> f32."""
    bits = capi.f32_to_bf16_trunc(a)
    return bits, (bits.astype(np.uint32) << 16).view(np.float32)


def make_weights(seed, E, d, f, f_s=0, gated=False, w_std=0.02, router_std=None, bias=None,
                 outlier_frac=0.0):
    rng = np.random.default_rng(seed)
    n = lambda *s: rng.standard_normal(s, dtype=np.float32)
    W = dict(
        w_router=n(E, d) * (router_std if router_std is not None else w_std),
        w_gate=n(E, f, d) * w_std, w_up=n(E, f, d) * w_std, w_down=n(E, d, f) * w_std)
    if f_s:
        W.update(s_gate=n(f_s, d) * w_std, s_up=n(f_s, d) * w_std, s_down=n(d, f_s) * w_std)
        if gated:
            W["shared_gate"] = n(d) * w_std
    if bias is not None:
        W["router_bias"] = np.asarray(bias, dtype=np.float32)
    if outlier_frac > 0:
        for name in ("w_gate", "w_up", "w_down"):
            a = W[name].reshape(-1, W[name].shape[-1])
            rows = rng.choice(a.shape[0], size=max(1, int(a.shape[0] * outlier_frac)),
                              replace=False)
            a[rows] *= 8.0
    return W


def build_pair(ora, W, top_k, convention, weight_dtype, max_tokens_hint=0, group_size=128):
    """Returns (oracle Layer on the stored values, capi Layer)."""
    proj = ["w_gate", "w_up", "w_down"] + (["s_gate", "s_up", "s_down"] if "s_gate" in W else [])
    stored, dev, scales = {}, {}, {}
    for name in proj:
        w = np.ascontiguousarray(W[name], dtype=np.float32)
        if weight_dtype == capi.WEIGHT_F32:
            stored[name] = dev[name] = w
        elif weight_dtype == capi.WEIGHT_BF16:
            dev[name], stored[name] = bf16_round_trip(w)
        elif weight_dtype == capi.WEIGHT_INT8_PER_GROUP:
            q, s = capi.quantize_per_group_i8(w, group_size)
            dev[name], scales[name] = q, s
            # the dequantised weight the reference computes with: q * scale of the element's group
            s_full = np.repeat(s, group_size, axis=-1)[..., :w.shape[-1]]
            stored[name] = (q.astype(np.float32) * s_full).astype(np.float32)
        else:
            q, s = capi.quantize_per_row_i8(w)
            dev[name], scales[name] = q, s
            stored[name] = (q.astype(np.float32) * s[..., None]).astype(np.float32)
    if weight_dtype == capi.WEIGHT_F32:
        router = W["w_router"]
    else:  # a bf16 checkpoint stores a bf16 router as well
        router = bf16_round_trip(W["w_router"])[1]
    common = dict(top_k=top_k, convention=convention, shared_gate=W.get("shared_gate"),
                  router_bias=W.get("router_bias"))
    oracle_layer = ora.Layer(w_router=router, w_gate=stored["w_gate"], w_up=stored["w_up"],
                             w_down=stored["w_down"], s_gate=stored.get("s_gate"),
                             s_up=stored.get("s_up"), s_down=stored.get("s_down"), **common)
    kw = {}
    if weight_dtype in (capi.WEIGHT_INT8_W8A16, capi.WEIGHT_INT8_PER_GROUP):
        if weight_dtype == capi.WEIGHT_INT8_PER_GROUP:
            kw["group_size"] = group_size
        kw.update(scale_gate=scales["w_gate"], scale_up=scales["w_up"],
                  scale_down=scales["w_down"])
        if "s_gate" in W:
            kw.update(s_scale_gate=scales["s_gate"], s_scale_up=scales["s_up"],
                      s_scale_down=scales["s_down"])
    gpu_layer = capi.Layer(w_router=router, w_gate=dev["w_gate"], w_up=dev["w_up"],
                           w_down=dev["w_down"], s_gate=dev.get("s_gate"), s_up=dev.get("s_up"),
                           s_down=dev.get("s_down"), weight_dtype=weight_dtype,
                           max_tokens_hint=max_tokens_hint, **common, **kw)
    return oracle_layer, gpu_layer


def make_tokens(seed, T, d, bf16=True):
    x = np.random.default_rng(seed).standard_normal((T, d), dtype=np.float32)
    return bf16_round_trip(x)[1] if bf16 else x


def rel_err(a, ref):
    """max|a - ref| / max|ref| -- the layer-output metric of the parity bar."""
    ref = np.asarray(ref, dtype=np.float64)
    return float(np.abs(np.asarray(a, dtype=np.float64) - ref).max() / np.abs(ref).max())


def bf16_rne(a):
    """f32 -> nearest-even bf16 -> f32 (the rounding the expert kernels apply to h)."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = u + 0x7FFF + ((u >> 16) & 1)
    return ((u >> 16) << 16).astype(np.uint32).view(np.float32)


FLIP_WINDOW = 2.0 ** -18  # relative distance from a bf16 rounding midpoint that counts as fragile


def _fragile_ulp(v, moved_by=0.0):
    """Per element: one bf16 ulp of v where v (an f32 array) lies within FLIP_WINDOW (relative) plus
    `moved_by` (absolute, per element) of the midpoint between two bf16 values -- there two
    computations of v that differ by that much may round to different bf16 neighbours -- and 0
    elsewhere."""
    low = (v.view(np.uint32) & 0xFFFF).astype(np.float64)          # position between two bf16 values
    expo = np.floor(np.log2(np.maximum(np.abs(v).astype(np.float64), 2.0 ** -126)))
    window = FLIP_WINDOW * 2.0 ** 23 + np.asarray(moved_by, dtype=np.float64) / 2.0 ** (expo - 23)
    fragile = np.abs(low - 0x8000) <= window
    return np.where(fragile, 2.0 ** (expo - 7), 0.0)


def emulate_bf16_kernels(oL, x, idx, w, with_slack=False, y_bf16=False, ys_bf16=False, split=None):
    """NumPy model of the bf16/int8 HIP path's arithmetic on the oracle layer's stored
    weights: exact products with wide accumulation, gate/up rounded to f32, h = silu(g)*u in
    f32 rounded to bf16 (nearest even), f32 combine with separate multiply and add.  The GPU
    result must sit within ~1e-3 of this model (difference: f32 accumulation order); the
    distance of either from the all-f64 reference is the bf16 rounding of h, ~2e-3 at real
    layer sizes.

    `y_bf16` / `ys_bf16`: the routed / shared expert outputs travel to the combine as bf16 (what
    `capi.plan_batch` reports for the batch): every expert output is rounded to bf16 (nearest even)
    before it is weighted.  `split` ([T, k, ceil(d / 256)], `Layer.last_down_split`): where the
    down launch cut a tile into S ranges of its 64-k stages, the output of that 256-column block is
    the f32 sum, in range order, of S partial sums, each rounded on its own.

    One more difference cannot be bounded by a relative figure: where silu(g)*u lies within a
    few f32 ulps of the midpoint between two bf16 values, the kernel (hardware exp2 / rcp, another
    summation order) and this model may round h to different neighbours, which moves that h by a
    whole bf16 ulp.  With a short down projection one such flip shows: the case E=40, k=3, d=128,
    f=96, T=700 has exactly one, and two variants of this model (silu through f32 or f64 exp)
    differ there by 1.954e-3 of the token's largest output, the same figure the kernel showed.
    `with_slack` also returns, per token, the largest output change that flips of the fragile h
    elements (within FLIP_WINDOW of a midpoint, about 0.2 % of all) can cause:
    sum over slots w * sum over fragile j max_n |W_d[n, j]| * ulp_bf16(h_j); and, for outputs that
    travel as bf16, of the fragile expert outputs themselves: max over n of the sum over slots of
    w * ulp_bf16(y[n]) (y, or the partial sum of a split block, near a rounding midpoint)."""
    T, d = x.shape
    out = np.zeros((T, d), dtype=np.float32)
    slack = np.zeros(T, dtype=np.float64)

    def expert(g, u, dn, xv, round_y, parts):
        gg = (g.astype(np.float64) @ xv).astype(np.float32)
        uu = (u.astype(np.float64) @ xv).astype(np.float32)
        hv = (gg / (np.float32(1) + np.exp(-gg, dtype=np.float32))) * uu
        h = bf16_rne(hv)
        low = (hv.view(np.uint32) & 0xFFFF).astype(np.int64)   # position between two bf16 values
        fragile = np.abs(low - 0x8000) <= FLIP_WINDOW * 2.0 ** 23
        bump = 0.0
        h_ulp = np.zeros(hv.shape, dtype=np.float64)  # what a flip moves each fragile h by
        if fragile.any():
            ulp = 2.0 ** (np.floor(np.log2(np.abs(hv[fragile]).astype(np.float64))) - 7)
            h_ulp[fragile] = ulp
            bump = float((np.abs(dn[:, fragile]).max(axis=0) * ulp).sum())
        h64 = h.astype(np.float64)
        if not round_y:
            return (dn.astype(np.float64) @ h64).astype(np.float32), bump, None
        # bf16 outputs: per 256-column block, S partial sums over ranges of 64-k stages
        f = h.shape[0]
        nst = (f + 63) // 64
        y = np.zeros(d, dtype=np.float32)
        y_ulp = np.zeros(d, dtype=np.float64)
        parts = np.ones((d + 255) // 256, dtype=np.int64) if parts is None else parts
        for S_ in np.unique(parts):
            cols = np.repeat(parts == S_, 256)[:d]
            acc = np.zeros(int(cols.sum()), dtype=np.float32)
            for i in range(int(S_)):
                lo, hi = 64 * (nst * i // int(S_)), min(f, 64 * (nst * (i + 1) // int(S_)))
                part = (dn[cols, lo:hi].astype(np.float64) @ h64[lo:hi]).astype(np.float32)
                # (a flip of a fragile h moves the sum a little, which can carry it across a
                # rounding midpoint of its own)
                moved = np.abs(dn[cols, lo:hi]).astype(np.float64) @ h_ulp[lo:hi]
                y_ulp[cols] += _fragile_ulp(part, moved)
                acc = acc + bf16_rne(part)
            y[cols] = acc
        return y, bump, y_ulp

    for t in range(T):
        xv = x[t].astype(np.float64)
        y_allow = np.zeros(d, dtype=np.float64)
        for s_, e in enumerate(idx[t]):
            y, bump, y_ulp = expert(oL.w_gate[e], oL.w_up[e], oL.w_down[e], xv, y_bf16,
                                    None if split is None else split[t, s_].astype(np.int64))
            out[t] = out[t] + w[t, s_] * y
            slack[t] += abs(float(w[t, s_])) * bump
            if y_ulp is not None:
                y_allow += abs(float(w[t, s_])) * y_ulp
        if oL.f_s:
            sc = np.float32(1.0)
            if oL.convention == 1 and oL.shared_gate is not None:
                acc = float(oL.shared_gate.astype(np.float64) @ xv)
                sc = np.float32(1.0 / (1.0 + np.exp(-acc)))
            y, bump, y_ulp = expert(oL.s_gate, oL.s_up, oL.s_down, xv, ys_bf16, None)
            out[t] = out[t] + sc * y
            slack[t] += float(sc) * bump
            if y_ulp is not None:
                y_allow += float(sc) * y_ulp
        slack[t] += float(y_allow.max())
    return (out, slack) if with_slack else out
