"""The Fepopel decoder family, restated plainly on the CPU in float64: one function per mechanism,
whole sequences at once, no cache.  The GPU library's kernels and the engine are tested against
this file; it shares no code with them.

A model is a list of layers, each  x += N1b(mixer(N1(x)));  x += N2b(ff(N2(x)))  (an RMS norm
before and after every sublayer).  Mixers: latent attention (keys and values expanded from one
latent per token, one rotated key part shared by the heads, a learned sink in the softmax's
denominator, an output gate per head) and grouped-query attention inside chunks of the sequence
(query and key normed per head, scores capped by a tanh).  Feed-forwards: a gated one, or routed
experts beside a gated shared expert.  A span of layers may run several times over with the same
weights, a learned vector added to the stream before every pass.
"""
import math

import torch

F64 = torch.float64


def rms_norm(x, w, eps):
    x = x.to(F64)
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w.to(F64)


def rotate_pairs(v, pos, dims, base):
    """v [T, ..., n]: channels 2i and 2i+1 (i < dims/2) turn by pos * base^(-2i/dims)."""
    v = v.to(F64).clone()
    i = torch.arange(dims // 2, dtype=F64)
    ang = pos.to(F64)[:, None] * torch.tensor(base, dtype=F64) ** (-2.0 * i / dims)   # [T, dims/2]
    shape = [v.shape[0]] + [1] * (v.dim() - 2) + [dims // 2]
    c, s = ang.cos().view(shape), ang.sin().view(shape)
    a, b = v[..., 0:dims:2].clone(), v[..., 1:dims:2].clone()
    v[..., 0:dims:2] = a * c - b * s
    v[..., 1:dims:2] = b * c + a * s
    return v


def visible(i, j, chunk=0):
    """Whether the query at position i sees the key at position j."""
    return j <= i and (chunk <= 0 or i // chunk == j // chunk)


def attend(q, k, v, pos_q, scale, chunk=0, softcap=0.0, sink=None):
    """q [n, H, dk] at positions pos_q against keys k [T, G, dk] / values v [T, G, dv] at positions
    0..T-1 -> [n, H, dv].  Head h reads key head h // (H/G).  sink [H]: one more term exp(sink) in
    the denominator."""
    n, H, _ = q.shape
    T, G, _ = k.shape
    rep = H // G
    k, v = k.to(F64).repeat_interleave(rep, 1), v.to(F64).repeat_interleave(rep, 1)
    s = torch.einsum("ihd,jhd->hij", q.to(F64), k) * scale
    if softcap > 0:
        s = softcap * torch.tanh(s / softcap)
    i, j = torch.as_tensor(pos_q).long()[:, None], torch.arange(T)[None, :]
    seen = (j <= i) & ((i // chunk == j // chunk) if chunk > 0 else True)          # visible(i, j, chunk), all pairs at once
    s = s.masked_fill(~seen[None], -math.inf)
    mx = s.max(-1).values
    if sink is not None:
        mx = torch.maximum(mx, sink.to(F64)[:, None])
    e = torch.exp(s - mx[..., None])
    den = e.sum(-1)
    if sink is not None:
        den = den + torch.exp(sink.to(F64)[:, None] - mx)
    return torch.einsum("hij,jhd->ihd", e / den[..., None], v)


def latent_attention(h, m, t, pos):
    """h [T, W] -> [T, W].  m: the mixer's sizes and constants; t: its tensors by short name."""
    T = h.shape[0]
    H, dk, dr, dv, rk = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    h = h.to(F64)
    q = (h @ t["q"].to(F64).T).view(T, H, dk + dr)
    low = h @ t["dkv"].to(F64).T
    c = rms_norm(low[:, :rk], t["dkv.norm"], m["eps"])                              # the latent
    k_rot = rotate_pairs(low[:, rk:], pos, m["rot"]["dims"], m["rot"]["base"])      # [T, dr], shared by the heads
    q_rot = rotate_pairs(q[..., dk:], pos, m["rot"]["dims"], m["rot"]["base"])
    k = torch.cat([(c @ t["uk"].to(F64).T).view(T, H, dk), k_rot[:, None, :].expand(T, H, dr)], -1)
    v = (c @ t["uv"].to(F64).T).view(T, H, dv)
    o = attend(torch.cat([q[..., :dk], q_rot], -1), k, v, pos, m["scale"], sink=t["sink"])
    gate = torch.sigmoid(h @ t["g"].to(F64).T)                                      # [T, H]
    return (o * gate[..., None]).reshape(T, H * dv) @ t["o"].to(F64).T


def chunk_attention(h, m, t, pos):
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    h = h.to(F64)
    q = rms_norm((h @ t["q"].to(F64).T).view(T, H, dk), t["q.norm"], m["eps"])
    k = rms_norm((h @ t["k"].to(F64).T).view(T, G, dk), t["k.norm"], m["eps"])
    v = (h @ t["v"].to(F64).T).view(T, G, dv)
    o = attend(q, k, v, pos, m["scale"], chunk=m["mask"]["size"], softcap=m["softcap"])
    return o.reshape(T, H * dv) @ t["o"].to(F64).T


def dense_ff(h, t):
    h = h.to(F64)
    g = h @ t["gate"].to(F64).T
    return (g * torch.sigmoid(g) * (h @ t["up"].to(F64).T)) @ t["down"].to(F64).T


def squared_relu_ff(h, up, down):
    return torch.relu(h.to(F64) @ up.to(F64).T).pow(2) @ down.to(F64).T


def route(h, w_router, top, scale):
    """(chosen experts [T, top], their weights [T, top])."""
    s = torch.softmax(h.to(F64) @ w_router.to(F64).T, -1)
    val, idx = s.topk(top, -1)
    return idx, val / (val.sum(-1, keepdim=True) + 1e-20) * scale


def experts_ff(h, mlp, t):
    r = mlp["router"]
    idx, wt = route(h, t["router"], r["top"], r["scale"])
    out = torch.zeros(h.shape[0], t["e0.down"].shape[0], dtype=F64)
    for e in range(r["experts"]):
        rows, slot = (idx == e).nonzero(as_tuple=True)
        if rows.numel():
            out[rows] += wt[rows, slot][:, None] * squared_relu_ff(h[rows], t[f"e{e}.up"], t[f"e{e}.down"])
    if mlp.get("shared"):
        g = torch.sigmoid(h.to(F64) @ t["shared.sg"].to(F64).T)                 # [T, 1]
        out = out + g * squared_relu_ff(h, t["shared.up"], t["shared.down"])
    return out


def sub(state, prefix):
    return {k[len(prefix):]: v for k, v in state.items() if k.startswith(prefix)}


def layer_runs(cfg):
    """The order in which layers run: (layer, pass) pairs; pass is None outside the repeated span."""
    n, loop = len(cfg["layers"]), cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    a, b, times = loop["start"], loop["stop"], loop["times"]
    return ([(i, None) for i in range(a)] + [(i, p) for p in range(times) for i in range(a, b)]
            + [(i, None) for i in range(b, n)])


def forward(cfg, state, tokens, layer_out=None):
    """tokens [T] of one sequence -> logits [T, vocab] (float64)."""
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    pos = torch.arange(tokens.numel())
    eps = cfg["norm"]["eps"]
    x = state["embed"].to(F64)[tokens] * cfg["embedding"]["scale"]
    loop = cfg.get("loop")
    for i, p in layer_runs(cfg):
        if p is not None and i == loop["start"]:
            x = x + state["loop.step"].to(F64)[p]
        l, pre = cfg["layers"][i], f"l{i}."
        m = dict(l["mixer"], eps=eps)
        mix = latent_attention if l["type"] == "latent_attention" else chunk_attention
        if l["type"] not in ("latent_attention", "attention"):
            raise ValueError(l["type"])
        x = x + rms_norm(mix(rms_norm(x, state[pre + "norm1"], eps), m, sub(state, pre + "mix."), pos),
                         state[pre + "norm1b"], eps)
        mlp = l.get("mlp")
        if mlp:
            h = rms_norm(x, state[pre + "norm2"], eps)
            t = sub(state, pre + "mlp.")
            y = dense_ff(h, t) if mlp["kind"] == "dense" else experts_ff(h, mlp, t)
            x = x + rms_norm(y, state[pre + "norm2b"], eps)
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
    if cfg.get("loop"):
        st["loop.step"] = rn(cfg["loop"]["times"], W, s=0.5)
    for i, l in enumerate(cfg["layers"]):
        m, p = l["mixer"], f"l{i}."
        H, dk, dv = m["heads"], m["dim"], m["vdim"]
        st[p + "norm1"], st[p + "norm1b"] = 1 + rn(W, s=0.1), 1 + rn(W, s=0.1)
        if l["type"] == "latent_attention":
            rk, dr = m["kv_rank"], m["rot_dim"]
            st[p + "mix.q"], st[p + "mix.dkv"] = rn(H * (dk + dr), W, s=W ** -0.5), rn(rk + dr, W, s=W ** -0.5)
            st[p + "mix.dkv.norm"] = 1 + rn(rk, s=0.1)
            st[p + "mix.uk"], st[p + "mix.uv"] = rn(H * dk, rk, s=rk ** -0.5), rn(H * dv, rk, s=rk ** -0.5)
            st[p + "mix.sink"], st[p + "mix.g"] = rn(H), rn(H, W, s=W ** -0.5)
        else:
            G = m["kv_heads"]
            st[p + "mix.q"], st[p + "mix.k"] = rn(H * dk, W, s=W ** -0.5), rn(G * dk, W, s=W ** -0.5)
            st[p + "mix.v"] = rn(G * dv, W, s=W ** -0.5)
            st[p + "mix.q.norm"], st[p + "mix.k.norm"] = 1 + rn(dk, s=0.1), 1 + rn(dk, s=0.1)
        st[p + "mix.o"] = rn(W, H * dv, s=(H * dv) ** -0.5)
        mlp = l.get("mlp")
        if not mlp:
            continue
        st[p + "norm2"], st[p + "norm2b"] = 1 + rn(W, s=0.1), 1 + rn(W, s=0.1)
        if mlp["kind"] == "dense":
            F = mlp["ff"]
            st[p + "mlp.gate"], st[p + "mlp.up"], st[p + "mlp.down"] = rn(F, W, s=W ** -0.5), rn(F, W, s=W ** -0.5), rn(W, F, s=F ** -0.5)
            continue
        E, F = mlp["router"]["experts"], mlp["expert"]["ff"]
        st[p + "mlp.router"] = rn(E, W, s=2 * W ** -0.5)
        for e in range(E):
            st[p + f"mlp.e{e}.up"], st[p + f"mlp.e{e}.down"] = rn(F, W, s=W ** -0.5), rn(W, F, s=F ** -0.5)
        if mlp.get("shared"):
            Fs = mlp["shared"]["ff"]
            st[p + "mlp.shared.up"], st[p + "mlp.shared.down"] = rn(Fs, W, s=W ** -0.5), rn(W, Fs, s=Fs ** -0.5)
            st[p + "mlp.shared.sg"] = rn(1, W, s=W ** -0.5)
    return st
