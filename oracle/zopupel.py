"""The Zopupel decoder family, restated plainly on the CPU in float64: one function per mechanism,
whole sequences at once, no cache.  The GPU library's kernels and the engine are tested against
this file; it shares no code with them.

A model is a list of layers, each  x += m N1b(mixer(N1(x)));  x += m N2b(ff(N2(x)))  with one
constant m for the whole model and an RMS norm before and after every sublayer.  Two mixers, both
causal grouped-query attention over every earlier token with rotate-half rotary positions on the
leading channels of a head:

* differential attention: every head holds two score maps over the same values; the second map's
  output is subtracted, times one number per layer, and the head's difference is divided by its
  root mean square.  Frequencies divided by a constant.  A layer may read another layer's keys
  and values instead of projecting its own.
* attention whose values are its keys as projected: biases on the projections, query and key
  normed over the whole projection before rotation, frequencies blended along a ramp between
  fast and slow pairs, and a softmax whose denominator holds one more term of score 0.

The feed-forward is a set of routed experts (softmax over the chosen logits, a bias on the
router) beside a shared expert every token uses.
"""
import math

import torch

F64 = torch.float64


def rms_norm(x, w, eps):
    x = x.to(F64)
    y = x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)
    return y if w is None else y * w.to(F64)


def frequencies(rot):
    """(frequency of every pair [dims/2], factor of cos and sin) of a 'rot' block."""
    dims, base, sc = rot["dims"], float(rot["base"]), rot.get("scaling") or {}
    i = torch.arange(dims // 2, dtype=F64)
    f = torch.tensor(base, dtype=F64) ** (-2.0 * i / dims)
    if not sc:
        return f, 1.0
    factor = float(sc["factor"])
    if "original" not in sc:                      # every pair slowed by the same factor
        return f / factor, 1.0

    def pair_of(turns):
        return dims * math.log(sc["original"] / (2 * math.pi * turns)) / (2 * math.log(base))

    lo = max(math.floor(pair_of(sc["fast"])), 0)
    hi = min(math.ceil(pair_of(sc["slow"])), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return f / factor * ramp + f * (1 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_half(v, pos, rot):
    """v [T, heads, n]: channel i pairs with channel i + dims/2 (i < dims/2); the rest pass."""
    dims = rot["dims"]
    if dims == 0:
        return v.to(F64)
    f, mag = frequencies(rot)
    ang = torch.as_tensor(pos).to(F64)[:, None] * f                     # [T, dims/2]
    c, s = (ang.cos() * mag)[:, None, :], (ang.sin() * mag)[:, None, :]
    v = v.to(F64).clone()
    a, b = v[..., :dims // 2].clone(), v[..., dims // 2:dims].clone()
    v[..., :dims // 2] = a * c - b * s
    v[..., dims // 2:dims] = b * c + a * s
    return v


def causal_softmax(s, pos_q, extra_one=False):
    """s [H, n, T] scores of queries at pos_q against keys 0..T-1 -> weights; extra_one: the
    denominator holds one more term exp(0)."""
    T = s.shape[-1]
    seen = torch.arange(T)[None, :] <= torch.as_tensor(pos_q).long()[:, None]
    s = s.masked_fill(~seen[None], -math.inf)
    mx = s.max(-1, keepdim=True).values
    if extra_one:
        mx = mx.clamp_min(0.0)
    e = torch.exp(s - mx)
    den = e.sum(-1, keepdim=True)
    if extra_one:
        den = den + torch.exp(-mx)
    return e / den


def diff_lambda(t, diff):
    """exp(lq1 . lk1) - exp(lq2 . lk2) + diff, in float32 as the layer's one number."""
    a = (t["lq1"].float() * t["lk1"].float()).sum()
    b = (t["lq2"].float() * t["lk2"].float()).sum()
    return float(torch.exp(a) - torch.exp(b) + diff)


def diff_keys_values(h, m, t, pos):
    """The keys (rotated, [T, G, 2, dk]) and values ([T, G, dv]) a differential layer caches."""
    T = h.shape[0]
    G, dk, dv = m["kv_heads"], m["dim"], m["vdim"]
    k = (h.to(F64) @ t["k"].to(F64).T).view(T, G * 2, dk)
    k = rotate_half(k, pos, m["rot"]).view(T, G, 2, dk)
    return k, (h.to(F64) @ t["v"].to(F64).T).view(T, G, dv)


def diff_attention(h, m, t, pos, kv=None):
    """h [T, W] -> [T, W].  kv: another layer's (keys, values) to read instead of this one's."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rotate_half((h.to(F64) @ t["q"].to(F64).T).view(T, H * 2, dk), pos, m["rot"]).view(T, H, 2, dk)
    k, v = kv if kv is not None else diff_keys_values(h, m, t, pos)
    rep = H // G
    k, v = k.repeat_interleave(rep, 1), v.repeat_interleave(rep, 1)     # head h reads kv head h // rep
    lam = diff_lambda(t, m["diff"])
    out = []
    for mp in range(2):
        s = torch.einsum("ihd,jhd->hij", q[:, :, mp], k[:, :, mp]) * m["scale"]
        out.append(torch.einsum("hij,jhd->ihd", causal_softmax(s, pos), v))
    o = out[0] - lam * out[1]
    o = rms_norm(o, None, m["eps"]) * (1.0 - m["diff"])
    return o.reshape(T, H * dv) @ t["o"].to(F64).T


def keyvalue_attention(h, m, t, pos):
    """Attention whose values are its keys as projected.  h [T, W] -> [T, W]."""
    T = h.shape[0]
    H, G, dk = m["heads"], m["kv_heads"], m["dim"]
    h = h.to(F64)
    q = h @ t["q"].to(F64).T + t["q.b"].to(F64)
    k = h @ t["k"].to(F64).T + t["k.b"].to(F64)
    v = k.view(T, G, dk)
    q = rotate_half(rms_norm(q, t["q.norm"], m["eps"]).view(T, H, dk), pos, m["rot"])
    k = rotate_half(rms_norm(k, t["k.norm"], m["eps"]).view(T, G, dk), pos, m["rot"])
    rep = H // G
    s = torch.einsum("ihd,jhd->hij", q, k.repeat_interleave(rep, 1)) * m["scale"]
    o = torch.einsum("hij,jhd->ihd", causal_softmax(s, pos, extra_one=True), v.repeat_interleave(rep, 1))
    return o.reshape(T, H * dk) @ t["o"].to(F64).T + t["o.b"].to(F64)


def gated_ff(h, gate, up, down):
    g = h.to(F64) @ gate.to(F64).T
    return (g * torch.sigmoid(g) * (h.to(F64) @ up.to(F64).T)) @ down.to(F64).T


def route(h, w_router, b_router, top):
    """(chosen experts [T, top], their weights [T, top]): softmax over the chosen logits only."""
    z = h.to(F64) @ w_router.to(F64).T + b_router.to(F64)
    val, idx = z.topk(top, -1)
    return idx, torch.softmax(val, -1)


def experts_ff(h, mlp, t):
    r = mlp["router"]
    idx, wt = route(h, t["router"], t["router.b"], r["top"])
    out = torch.zeros(h.shape[0], t["e0.down"].shape[0], dtype=F64)
    for e in range(r["experts"]):
        rows, slot = (idx == e).nonzero(as_tuple=True)
        if rows.numel():
            out[rows] += wt[rows, slot][:, None] * gated_ff(h[rows], t[f"e{e}.gate"], t[f"e{e}.up"], t[f"e{e}.down"])
    if mlp.get("shared"):
        out = out + gated_ff(h, t["shared.gate"], t["shared.up"], t["shared.down"])
    return out


def sub(state, prefix):
    return {k[len(prefix):]: v for k, v in state.items() if k.startswith(prefix)}


def forward(cfg, state, tokens, layer_out=None):
    """tokens [T] of one sequence -> logits [T, vocab] (float64)."""
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    pos = torch.arange(tokens.numel())
    eps, mult = cfg["norm"]["eps"], cfg["residual_mult"]
    x = state["embed"].to(F64)[tokens]
    kept = {}                                            # keys and values of the layers others read
    for i, l in enumerate(cfg["layers"]):
        pre = f"l{i}."
        m, t = dict(l["mixer"], eps=eps), sub(state, pre + "mix.")
        h = rms_norm(x, state[pre + "norm1"], eps)
        if l["type"] == "attention":
            src = m.get("kv_from")
            if src is None:
                kept[i] = diff_keys_values(h, m, t, pos)
            y = diff_attention(h, m, t, pos, kv=kept[i if src is None else src])
        elif l["type"] == "attention_2":
            y = keyvalue_attention(h, m, t, pos)
        else:
            raise ValueError(l["type"])
        x = x + mult * rms_norm(y, state[pre + "norm1b"], eps)
        mlp = l.get("mlp")
        if mlp:
            y = experts_ff(rms_norm(x, state[pre + "norm2"], eps), mlp, sub(state, pre + "mlp."))
            x = x + mult * rms_norm(y, state[pre + "norm2b"], eps)
        if layer_out is not None:
            layer_out.append(x.clone())
    return rms_norm(x, state["final.norm"], eps) @ state["head"].to(F64).T


def random_tensors(cfg, seed=0):
    """Seeded random tensors (bfloat16 values, as float32) under the checkpoint's names."""
    g = torch.Generator().manual_seed(seed)

    def rn(*shape, s=1.0):
        return (torch.randn(*shape, generator=g) * s).to(torch.bfloat16).float()

    W, st = cfg["width"], {}
    st["embed"], st["head"], st["final.norm"] = rn(cfg["vocab"], W), rn(cfg["vocab"], W, s=W ** -0.5), 1 + rn(W, s=0.1)
    for i, l in enumerate(cfg["layers"]):
        m, p = l["mixer"], f"l{i}."
        H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        st[p + "norm1"], st[p + "norm1b"] = 1 + rn(W, s=0.1), 1 + rn(W, s=0.1)
        if l["type"] == "attention":
            st[p + "mix.q"] = rn(H * 2 * dk, W, s=W ** -0.5)
            if m.get("kv_from") is None:
                st[p + "mix.k"], st[p + "mix.v"] = rn(G * 2 * dk, W, s=W ** -0.5), rn(G * dv, W, s=W ** -0.5)
            for n in ("lq1", "lk1", "lq2", "lk2"):
                st[p + "mix." + n] = rn(dk, s=0.3)
        else:
            st[p + "mix.q"], st[p + "mix.k"] = rn(H * dk, W, s=W ** -0.5), rn(G * dk, W, s=W ** -0.5)
            st[p + "mix.q.b"], st[p + "mix.k.b"], st[p + "mix.o.b"] = rn(H * dk, s=0.3), rn(G * dk, s=0.3), rn(W, s=0.3)
            st[p + "mix.q.norm"], st[p + "mix.k.norm"] = 1 + rn(H * dk, s=0.1), 1 + rn(G * dk, s=0.1)
        st[p + "mix.o"] = rn(W, H * dv, s=(H * dv) ** -0.5)
        mlp = l.get("mlp")
        if not mlp:
            continue
        st[p + "norm2"], st[p + "norm2b"] = 1 + rn(W, s=0.1), 1 + rn(W, s=0.1)
        E, F = mlp["router"]["experts"], mlp["expert"]["ff"]
        st[p + "mlp.router"], st[p + "mlp.router.b"] = rn(E, W, s=2 * W ** -0.5), rn(E, s=0.5)
        for e in range(E):
            st[p + f"mlp.e{e}.gate"], st[p + f"mlp.e{e}.up"] = rn(F, W, s=W ** -0.5), rn(F, W, s=W ** -0.5)
            st[p + f"mlp.e{e}.down"] = rn(W, F, s=F ** -0.5)
        if mlp.get("shared"):
            Fs = mlp["shared"]["ff"]
            st[p + "mlp.shared.gate"], st[p + "mlp.shared.up"] = rn(Fs, W, s=W ** -0.5), rn(Fs, W, s=W ** -0.5)
            st[p + "mlp.shared.down"] = rn(W, Fs, s=Fs ** -0.5)
    return st
