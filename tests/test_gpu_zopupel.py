"""The Zopupel decoder family on the GPU against the plain CPU restatement in oracle/zopupel.py:
every mechanism alone through its entry point, then whole models through the engine (prompts
whole, token by token, in portions, in mixed batches, over reused slots and pages) and through
the worker and scheduler.  Small random models of several shapes; where random weights would hide
a fault (one far key among many, the unit term of the denominator, the first tokens) the inputs
are made so that it shows."""
import math

import pytest
import torch

from oracle import zopupel as Z

pytestmark = pytest.mark.gpu

DEV = "cuda"
PAGE = 16
F64 = torch.float64


def dev(t, dtype=None):
    return t.to(dtype or t.dtype).contiguous().to(DEV)


def i32(x):
    return torch.tensor(x, dtype=torch.int32, device=DEV)


def rel(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return ((a - b).pow(2).mean().sqrt() / b.pow(2).mean().sqrt().clamp_min(1e-30)).item()


# ------------------------------------------------------------------ model shapes
def blend(factor=4.0, original=64, fast=8.0, slow=1.0):
    return {"factor": factor, "original": original, "fast": fast, "slow": slow}


def keyval(heads=4, kv_heads=2, dim=8, rot=6, base=10000.0, scale=0.4, scaling="default", mlp="default"):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=scale,
             rot={"dims": rot, "base": base, "scaling": blend() if scaling == "default" else scaling})
    return {"type": "attention_2", "mixer": m, "mlp": experts() if mlp == "default" else mlp}


def diff(heads=4, kv_heads=2, dim=8, vdim=12, rot=4, base=5000.0, scale=0.5, d=0.3, factor=2.0, kv_from=None,
         mlp="default"):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale, diff=d,
             rot={"dims": rot, "base": base, "scaling": {"factor": factor}})
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m, "mlp": experts() if mlp == "default" else mlp}


def experts(n=4, top=2, ff=24, shared=20):
    out = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": n, "top": top}}
    if shared:
        out["shared"] = {"ff": shared}
    return out


def model_cfg(layers, width=32, vocab=80, eps=1e-5, mult=0.4):
    return {"architecture": "Zopupel", "width": width, "vocab": vocab, "norm": {"eps": eps}, "residual_mult": mult,
            "layers": layers}


SHAPES = {
    "two_kinds": model_cfg([keyval(), diff(), keyval(mlp=None), diff(kv_from=1)]),
    # sizes that divide nothing; every pair of sizes that may coincide made different; three heads on a
    # kv head; two layers reading the keys of one; a layer without feed-forward; all experts chosen
    "odd": model_cfg([diff(heads=6, kv_heads=2, dim=12, vdim=20, rot=6, d=0.55, factor=3.0, mlp=experts(3, 3, 10, 0)),
                      keyval(heads=3, kv_heads=3, dim=10, rot=10, base=300.0, scaling=blend(2.5, 40, 5.0, 0.5), mlp=None),
                      diff(heads=6, kv_heads=2, dim=12, vdim=20, rot=6, d=0.55, factor=3.0, kv_from=0),
                      keyval(heads=5, kv_heads=1, dim=14, rot=2, scale=0.2, mlp=experts(5, 3, 20, 12)),
                      diff(heads=6, kv_heads=2, dim=12, vdim=20, rot=6, d=0.55, factor=3.0, kv_from=0,
                           mlp=experts(7, 1, 9, 5))],
                     width=40, vocab=131, eps=1e-6, mult=0.7),
    # one head, one expert, factors of one, a constant of zero, every channel rotated or none
    "ones": model_cfg([keyval(heads=1, kv_heads=1, dim=4, rot=4, scale=1.0, scaling=blend(1.0, 16, 2.0, 1.0),
                              mlp=experts(1, 1, 8, 4)),
                       diff(heads=1, kv_heads=1, dim=6, vdim=6, rot=0, d=0.0, factor=1.0, scale=1.0, mlp=None),
                       keyval(heads=2, kv_heads=1, dim=4, rot=0, scaling=None, mlp=experts(2, 2, 8, 0))],
                      width=24, vocab=50, mult=1.0),
    # widths that are multiples of 32: bfloat16 serving takes the tiled linear kernels and the matrix cores
    "aligned": model_cfg([keyval(heads=4, kv_heads=2, dim=16, rot=8, mlp=experts(8, 2, 32, 64)),
                          diff(heads=4, kv_heads=1, dim=16, vdim=16, rot=16, mlp=experts(8, 2, 32, 64)),
                          diff(heads=4, kv_heads=1, dim=16, vdim=16, rot=16, kv_from=1, mlp=experts(8, 2, 32, 64))],
                         width=64, vocab=178),
    # heads wider than a wave, values wider than two tiles of columns, eight and more heads on a kv head
    "wide": model_cfg([keyval(heads=9, kv_heads=1, dim=72, rot=40), diff(heads=8, kv_heads=1, dim=72, vdim=136, rot=72),
                       keyval(heads=16, kv_heads=2, dim=130, rot=64)], width=48, vocab=64),
}


def build(cfg, dtype=torch.float32, seed=0, tiled=True, st=None, **eng_kw):
    from vllm_omni_draft_amd import config, weights
    from vllm_omni_draft_amd.seq_engine import SeqEngine, SeqEngineConfig
    st = st or Z.random_tensors(cfg, seed)
    mc = config.zopupel_config(cfg, {k: tuple(v.shape) for k, v in st.items()})
    w = weights.seq_from_state_dict(mc, st, DEV, dtype, tiled=tiled)
    kw = dict(max_seqs=4, max_tokens=1024)
    kw.update(eng_kw)
    return st, SeqEngine(w, SeqEngineConfig(**kw))


def prompt(cfg, n, seed=0):
    g = torch.Generator().manual_seed(1000 + seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


def fill_pages(rows, units, pages_of):
    """rows [n, units*d] of one sequence in slot 0 -> cache [pages, units, PAGE, d], written here
    (not through the library): token j lies in page pages_of[j // PAGE], row j % PAGE."""
    n, d = rows.shape[0], rows.shape[1] // units
    cache = torch.zeros(max(pages_of) + 1, units, PAGE, d, dtype=rows.dtype)
    for j in range(n):
        cache[pages_of[j // PAGE], :, j % PAGE] = rows[j].view(units, d)
    return cache.to(DEV)


def table(pages_of):
    bt = torch.zeros(2, len(pages_of), dtype=torch.int32, device=DEV)
    bt[0] = i32(pages_of)
    return bt


def plain_attention(q, k, v, pos, H, G, maps, scale, extra_one=False):
    """q [n, H*maps*dk] at positions pos against k [T, G*maps*dk], v [T, G*dv] -> [n, H*maps*dv]."""
    n, T = q.shape[0], k.shape[0]
    dk, dv = q.shape[1] // (H * maps), v.shape[1] // G
    q, k, v = q.to(F64).view(n, H, maps, dk), k.to(F64).view(T, G, maps, dk), v.to(F64).view(T, G, dv)
    rep = H // G
    out = torch.zeros(n, H, maps, dv, dtype=F64)
    for m in range(maps):
        s = torch.einsum("ihd,jhd->hij", q[:, :, m], k[:, :, m].repeat_interleave(rep, 1)) * scale
        out[:, :, m] = torch.einsum("hij,jhd->ihd", Z.causal_softmax(s, pos, extra_one), v.repeat_interleave(rep, 1))
    return out.view(n, H * maps * dv)


# ------------------------------------------------------------------ mechanisms alone
@pytest.mark.parametrize("H,G,maps,dk,dv,sink", [(4, 2, 2, 16, 16, False), (3, 1, 1, 12, 20, True), (2, 2, 2, 72, 136, False),
                                                 (9, 1, 2, 8, 8, True), (16, 2, 1, 8, 300, True), (6, 2, 2, 12, 20, False)])
@pytest.mark.parametrize("cdt", [torch.float32, torch.bfloat16])
def test_attention_with_several_maps_random(H, G, maps, dk, dv, sink, cdt):
    from vllm_omni_draft_amd import ops
    g = torch.Generator().manual_seed(H * 100 + dk + maps)
    n = 45
    q = torch.randn(n, H * maps * dk, generator=g)
    k, v = torch.randn(n, G * maps * dk, generator=g).to(cdt), torch.randn(n, G * dv, generator=g).to(cdt)
    pages = [5, 1, 3]                                  # pages out of order
    kc, vc, bt = fill_pages(k, G * maps, pages), fill_pages(v, G, pages), table(pages)
    sinks = torch.zeros(H * maps, device=DEV) if sink else None
    want = plain_attention(q, k, v, torch.arange(n), H, G, maps, 0.3, extra_one=sink)
    for rows in (list(range(n)), [n - 1], [0, 15, 16, 17, 31, 32, 44]):     # a prompt, one decoded row, a few rows
        for split in (True, False):
            got = ops.multimap_softmax_attention(dev(q[rows]), kc, vc, i32(rows), i32([0] * len(rows)), bt, H, G, maps,
                                                 dk, dv, 0.3, sinks=sinks, split=split)
            assert rel(got, want[rows]) < 3e-6, (len(rows), split)


def test_the_unit_term_takes_its_share():
    """All scores equal zero (a zero query): with one more term exp(0) in the denominator the row
    at position i returns the sum of its i + 1 values divided by i + 2; without it, their mean."""
    from vllm_omni_draft_amd import ops
    n, H, G, dk, dv = 40, 2, 1, 8, 4
    g = torch.Generator().manual_seed(3)
    k, v = torch.randn(n, G * dk, generator=g), torch.randn(n, G * dv, generator=g)
    pages = [2, 0, 1]
    kc, vc, bt = fill_pages(k, G, pages), fill_pages(v, G, pages), table(pages)
    q = torch.zeros(n, H * dk, device=DEV)
    csum = v.double().cumsum(0)
    for rows in (list(range(n)), [0], [n - 1]):
        for sink, extra in ((torch.zeros(H, device=DEV), 1), (None, 0)):
            got = ops.multimap_softmax_attention(q[rows], kc, vc, i32(rows), i32([0] * len(rows)), bt, H, G, 1, dk, dv,
                                                 1.0, sinks=sink).view(len(rows), H, dv)
            for a, i in enumerate(rows):
                for h in range(H):
                    assert rel(got[a, h], csum[i] / (i + 1 + extra)) < 1e-6, (i, h, extra)


@pytest.mark.parametrize("cdt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("maps", [1, 2])
def test_a_far_key_among_hundreds(cdt, maps):
    """700 keys; the first map's query of head 0 points at key 3 and the second map's at key 650, so
    that each takes nearly all the weight of its own map only; every other head spreads out."""
    from vllm_omni_draft_amd import ops
    n, H, G, dk, dv = 700, 2, 1, 16, 8
    g = torch.Generator().manual_seed(11)
    k = torch.randn(n, G * maps * dk, generator=g)
    v = torch.randn(n, G * dv, generator=g).to(cdt)
    k = (k / k.view(n, G * maps, dk).norm(dim=-1).repeat_interleave(dk, 1)).to(cdt)     # unit keys
    pages = list(range(44))[::-1]
    kc, vc, bt = fill_pages(k, G * maps, pages), fill_pages(v, G, pages), table(pages)
    q = torch.randn(3, H * maps * dk, generator=g) * 0.1
    targets = [3, 650][:maps]
    for m, j in enumerate(targets):
        q[:, m * dk:(m + 1) * dk] = 60.0 * k[j].float().view(G * maps, dk)[m]
    rows = [699, 660, 652]
    want = plain_attention(q, k, v, torch.tensor(rows), H, G, maps, 1.0)
    got = ops.multimap_softmax_attention(dev(q), kc, vc, i32(rows), i32([0] * 3), bt, H, G, maps, dk, dv, 1.0)
    assert rel(got, want) < 3e-6
    for m, j in enumerate(targets):
        assert rel(got.view(3, H, maps, dv)[:, 0, m], v[j].float().expand(3, dv)) < 1e-3, (m, j)


@pytest.mark.parametrize("nq,nk,dk,G,dv,norm,rot,from_key,bias", [
    (4, 2, 16, 2, 16, "full", 8, True, True), (6, 4, 12, 2, 20, "none", 6, False, False),
    (5, 5, 10, 5, 10, "head", 10, True, False), (1, 1, 130, 1, 4, "full", 64, False, True),
    (8, 2, 8, 1, 24, "none", 0, False, True), (3, 3, 72, 3, 72, "full", 2, True, True)])
@pytest.mark.parametrize("wdt", [torch.float32, torch.bfloat16])
def test_preparation_in_one_launch(nq, nk, dk, G, dv, norm, rot, from_key, bias, wdt):
    """Bias, norm, rotary turn and the append against the plain pieces; the cached values of a layer
    whose values are its keys are the keys after their bias, before norm and turn."""
    from vllm_omni_draft_amd import ops
    g = torch.Generator().manual_seed(nq * 10 + dk)
    n, eps = 37, 1e-5
    pos = list(range(5, 5 + n))
    pages = [4, 0, 2]
    q, k = torch.randn(n, nq * dk, generator=g), torch.randn(n, nk * dk, generator=g)
    v = None if from_key else torch.randn(n, G * dv, generator=g)
    rnd = lambda *s: (torch.randn(*s, generator=g) * 0.5).to(wdt)
    qb, kb = (rnd(nq * dk), rnd(nk * dk)) if bias else (None, None)
    wn = {"full": (1 + rnd(nq * dk), 1 + rnd(nk * dk)), "head": (1 + rnd(dk), 1 + rnd(dk)), "none": (None, None)}[norm]
    rot_cfg = {"dims": rot, "base": 777.0, "scaling": blend(3.0, 32, 4.0, 0.5)}
    f, mag = Z.frequencies(rot_cfg) if rot else (None, 1.0)
    kc = torch.zeros(5, nk, PAGE, dk, dtype=wdt, device=DEV)
    vc = torch.zeros(5, G, PAGE, dv, dtype=wdt, device=DEV)
    gq, gk = ops.attn_prep(dev(q), dev(k), dev(v) if v is not None else None, dk, G, dv, i32(pos), i32([0] * n),
                           table(pages), kc, vc, q_bias=dev(qb) if bias else None, k_bias=dev(kb) if bias else None,
                           norm=norm, q_norm_w=dev(wn[0]) if wn[0] is not None else None,
                           k_norm_w=dev(wn[1]) if wn[1] is not None else None, eps=eps, rot_dims=rot,
                           inv_freq=dev(f) if rot else None, mag=mag)

    def plain(x, b, w, units):
        x = x.to(F64) + (b.to(F64) if b is not None else 0)
        raw = x.clone()
        if norm == "full":
            x = Z.rms_norm(x, w, eps)
        elif norm == "head":
            x = Z.rms_norm(x.view(n, units, dk), w, eps).reshape(n, units * dk)
        return Z.rotate_half(x.view(n, units, dk), torch.tensor(pos), rot_cfg).reshape(n, units * dk), raw

    wq, _ = plain(q, qb, wn[0], nq)
    wk, raw_k = plain(k, kb, wn[1], nk)
    assert rel(gq, wq) < 2e-6 and rel(gk, wk) < 2e-6
    wv = raw_k if from_key else v.to(F64)
    tol = 2e-6 if wdt == torch.float32 else 6e-3
    for a, p in enumerate(pos):
        pg = pages[p // PAGE]
        assert rel(kc[pg, :, p % PAGE].reshape(-1), wk[a]) < tol and rel(vc[pg, :, p % PAGE].reshape(-1), wv[a]) < tol, p
    # a layer that reads another layer's keys prepares its queries only
    gq2, none = ops.attn_prep(dev(q), None, None, dk, G, dv, i32(pos), None, None, None, None,
                              q_bias=dev(qb) if bias else None, norm=norm,
                              q_norm_w=dev(wn[0]) if wn[0] is not None else None, eps=eps, rot_dims=rot,
                              inv_freq=dev(f) if rot else None, mag=mag)
    assert none is None and torch.equal(gq2, gq)


def test_frequencies_of_both_scalings():
    """The reader's frequencies against the plain ones, for the divided and the blended kind, and a
    ramp that is not flat: some pair keeps its frequency, some pair is slowed by the whole factor."""
    from vllm_omni_draft_amd import config
    for rot in ({"dims": 16, "base": 10000.0, "scaling": {"factor": 2.0}}, {"dims": 6, "base": 50.0},
                {"dims": 32, "base": 1e4, "scaling": blend(8.0, 128, 16.0, 1.0)},
                {"dims": 10, "base": 300.0, "scaling": blend(2.5, 40, 5.0, 0.5)}):
        f, mag = config.rotary_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
        wf, wmag = Z.frequencies(rot)
        assert torch.equal(f, wf) and mag == wmag
    f, mag = Z.frequencies({"dims": 32, "base": 1e4, "scaling": blend(8.0, 128, 16.0, 1.0)})
    plain = torch.tensor(1e4, dtype=F64) ** (-torch.arange(16, dtype=F64) / 16)
    assert f[0] == plain[0] and abs(f[-1] / plain[-1] - 1 / 8) < 1e-12 and mag == 0.1 * math.log(8.0) + 1.0
    assert ((f / plain < 0.999) & (f / plain > 0.126)).any()


@pytest.mark.parametrize("H,dv", [(4, 16), (3, 20), (1, 136), (7, 5)])
def test_two_maps_put_together(H, dv):
    from vllm_omni_draft_amd import ops
    g = torch.Generator().manual_seed(H + dv)
    a = torch.randn(23, H, 2, dv, generator=g)
    lam, eps, scale = 0.37, 1e-5, 0.7
    t = a[:, :, 0].double() - lam * a[:, :, 1].double()
    want = (Z.rms_norm(t, None, eps) * scale).reshape(23, H * dv)
    y, yb = ops.diff_combine_rows(dev(a.reshape(23, -1)), lam, eps, scale, H, dv, bf16_copy=True)
    assert rel(y, want) < 3e-3 and torch.equal(yb.float(), y)            # (rounded to bfloat16 values with the copy)
    assert rel(ops.diff_combine_rows(dev(a.reshape(23, -1)), lam, eps, scale, H, dv), want) < 2e-6


def test_lambda_is_one_number_per_layer():
    from vllm_omni_draft_amd import config, weights
    cfg = model_cfg([diff(d=0.45, mlp=None)])
    st = Z.random_tensors(cfg, 2)
    w = weights.seq_from_state_dict(config.zopupel_config(cfg), st, DEV, torch.float32)
    want = Z.diff_lambda(Z.sub(st, "l0.mix."), 0.45)
    assert abs(w.layers[0].diff_lambda - want) < 1e-6 and abs(want - 0.45) > 1e-3


@pytest.mark.parametrize("E,K,top,wdt", [(5, 40, 3, torch.float32), (16, 1000, 2, torch.bfloat16), (130, 64, 7, torch.float32),
                                         (1, 24, 1, torch.float32), (6, 33, 6, torch.bfloat16)])
def test_router_with_a_bias(E, K, top, wdt):
    """The bias decides: it is made large enough to change which experts are chosen."""
    from vllm_omni_draft_amd import ops
    g = torch.Generator().manual_seed(E + K)
    x = torch.randn(19, K, generator=g).to(wdt).float()
    w, b = (torch.randn(E, K, generator=g) * K ** -0.5).to(wdt), torch.randn(E, generator=g) * 2
    idx, wt = Z.route(x, w.float(), b, top)
    if 1 < top < E:
        assert (Z.route(x, w.float(), torch.zeros(E), top)[0] != idx).any()
    se, sw, logits = ops.moe_route_rows_biased(dev(x), dev(w), dev(b), top)
    assert rel(logits, x.double() @ w.double().T + b.double()) < 5e-6
    assert torch.equal(se.cpu().long(), idx) and rel(sw, wt) < 2e-6
    assert torch.allclose(sw.sum(1).cpu(), torch.ones(19), atol=1e-6)


@pytest.mark.parametrize("W", [5, 72, 1000, 2048, 4100])
@pytest.mark.parametrize("wdt", [torch.float32, torch.bfloat16])
def test_scaled_residual_update_with_a_bias(W, wdt):
    from vllm_omni_draft_amd import ops
    g = torch.Generator().manual_seed(W)
    n, n_a, eps, mult = 7, 3, 1e-6, 0.3
    x, a, b = torch.randn(n, W, generator=g), torch.randn(n * n_a, W, generator=g), torch.randn(n, W, generator=g)
    wp, wn, ab = (1 + 0.1 * torch.randn(W, generator=g)).to(wdt), (1 + 0.1 * torch.randn(W, generator=g)).to(wdt), \
        torch.randn(W, generator=g).to(wdt)
    for bias, shared in ((ab, None), (None, b), (ab, b)):
        t = a.double().view(n, n_a, W).sum(1) + (bias.double() if bias is not None else 0) + \
            (shared.double() if shared is not None else 0)
        wx = x.double() + mult * Z.rms_norm(t, wp.float(), eps)
        gx = dev(x.clone())
        h = ops.residual_norm_scaled(gx, dev(a), dev(wp), mult, n_a=n_a, a_bias=dev(bias) if bias is not None else None,
                                     b=dev(shared) if shared is not None else None, w_next=dev(wn), eps=eps)
        assert rel(gx, wx) < 2e-6
        assert rel(h, Z.rms_norm(wx, wn.float(), eps)) < (2e-6 if wdt == torch.float32 else 4e-3)


# ------------------------------------------------------------------ whole models
@pytest.mark.parametrize("shape", list(SHAPES))
def test_prompt_logits_match_the_plain_model(shape):
    cfg = SHAPES[shape]
    st, eng = build(cfg)
    toks = prompt(cfg, 61)
    lo = []
    want = Z.forward(cfg, st, toks, lo)
    got, trace = eng.step([("a", toks, list(range(len(toks))))], layer_out=True)
    assert trace.shape[0] == len(lo) == len(cfg["layers"])
    for i, x in enumerate(lo):
        assert rel(trace[i], x) < 3e-6, f"residual after layer {i}"
    assert rel(got, want) < 3e-6


@pytest.mark.parametrize("shape,tiled", [("two_kinds", False), ("odd", False), ("aligned", True), ("aligned", False),
                                         ("wide", False)])
def test_bfloat16_serving_stays_close(shape, tiled):
    cfg = SHAPES[shape]
    st, eng = build(cfg, torch.bfloat16, tiled=tiled)
    toks = prompt(cfg, 50, 1)
    want = Z.forward(cfg, st, toks)
    got = eng.step([("a", toks, list(range(len(toks))))])
    # (a token whose router logits lie within bfloat16 rounding of each other may take another
    # expert than the plain model, and the tokens behind it feel that: most rows are close)
    rows = sorted(rel(got[r], want[r]) for r in range(len(toks)))
    assert rows[len(rows) // 2] < 2e-2 and rows[int(len(rows) * 0.9)] < 6e-2, rows[-5:]


@pytest.mark.parametrize("shape,dtype,tiled", [("two_kinds", torch.float32, True), ("odd", torch.float32, True),
                                               ("ones", torch.float32, True), ("wide", torch.float32, True),
                                               ("odd", torch.bfloat16, False), ("aligned", torch.bfloat16, True)])
def test_cut_anywhere_batched_anyhow(shape, dtype, tiled):
    """The logits of a position are the same however its prompt was cut into steps (down to two
    tokens and to single decoded tokens), whatever else shares the batch and whichever slot and
    pages the request got."""
    cfg = SHAPES[shape]
    st, eng = build(cfg, dtype, tiled=tiled)
    pa, pb, pc = prompt(cfg, 57, 1), prompt(cfg, 34, 2), prompt(cfg, 9, 3)
    whole = {}
    for name, p in (("a", pa), ("b", pb), ("c", pc)):
        whole[name] = eng.step([(name, p, list(range(len(p))))])
        eng.finish(name)
    if dtype == torch.float32:
        for name, p in (("a", pa), ("b", pb), ("c", pc)):
            assert rel(whole[name], Z.forward(cfg, st, p)) < 3e-6

    def same(x, y, what):
        # (few rows cut their keys over workgroups and merge them, many rows sweep them in one:
        # the two orders of summation differ in the last bits)
        assert rel(x, y) < (1e-5 if dtype == torch.float32 else 1e-2), what
    eng.step([("pad", prompt(cfg, 20, 9), [])])       # another slot and other pages than before
    got = torch.cat([eng.step([("a", [t], [0])]) for t in pa])
    same(got, whole["a"], "token by token")
    eng.finish("a")
    cuts_a = [0, 2, 4, 17, 19, 32, 33, 48, 57]
    cuts_b = [0, 16, 17, 18, 20, 34]
    got_a, got_b, got_c = [], [], []
    ia = ib = ic = 0
    while ia < len(cuts_a) - 1 or ib < len(cuts_b) - 1 or ic < len(pc):
        entries, kinds = [], []
        if ia < len(cuts_a) - 1:
            lo, hi = cuts_a[ia], cuts_a[ia + 1]
            entries.append(("a", pa[lo:hi], list(range(hi - lo))))
            kinds.append(got_a)
            ia += 1
        if ic < len(pc):
            entries.append(("c", pc[ic:ic + 1], [0]))
            kinds.append(got_c)
            ic += 1
        if ib < len(cuts_b) - 1:
            lo, hi = cuts_b[ib], cuts_b[ib + 1]
            entries.append(("b", pb[lo:hi], list(range(hi - lo))))
            kinds.append(got_b)
            ib += 1
        out = eng.step(entries)
        at = 0
        for (_, t, _), dst in zip(entries, kinds):
            dst.append(out[at:at + len(t)])
            at += len(t)
    same(torch.cat(got_a), whole["a"], "portions of a")
    same(torch.cat(got_b), whole["b"], "portions of b")
    same(torch.cat(got_c), whole["c"], "single tokens of c")


def test_slots_and_pages_are_used_again():
    cfg = SHAPES["two_kinds"]
    st, eng = build(cfg, max_seqs=3, max_tokens=12 * PAGE, max_seq_len=6 * PAGE)
    ref = {}
    for r in range(10):
        p = prompt(cfg, 20 + 7 * (r % 5), r)
        ref[r] = (p, Z.forward(cfg, st, p)[-1])
    live, nxt, done = {}, 0, 0
    while done < 10:
        while len(live) < 3 and nxt < 10:
            live[nxt] = 0
            nxt += 1
        entries = []
        for r in list(live):
            p = ref[r][0]
            n = min(len(p) - live[r], 13 if r % 2 else 1000)
            entries.append((str(r), p[live[r]:live[r] + n], [n - 1] if live[r] + n == len(p) else []))
            live[r] += n
        out = eng.step(entries)
        at = 0
        for rid, _, want in entries:
            if want:
                assert rel(out[at], ref[int(rid)][1]) < 3e-6, rid
                at += 1
                eng.finish(rid)
                del live[int(rid)]
                done += 1
    assert eng.free_slots == 3 and eng.cache.allocator.num_free == 12


def test_shared_keys_own_no_cache():
    cfg = SHAPES["odd"]
    _, eng = build(cfg)
    c = eng.cache
    assert sorted(c.k) == [0, 1, 3] and c.kv_source == {2: 0, 4: 0}
    assert c.keys_of(4) is c.k[0] and c.values_of(2) is c.v[0]
    assert tuple(c.k[0].shape[1:]) == (2 * 2, PAGE, 12) and tuple(c.v[0].shape[1:]) == (2, PAGE, 20)
    assert tuple(c.k[1].shape[1:]) == tuple(c.v[1].shape[1:]) == (3, PAGE, 10)


def test_a_step_larger_than_a_pass():
    cfg = SHAPES["two_kinds"]
    st, eng = build(cfg, max_rows=16)
    pa, pb = prompt(cfg, 45, 4), prompt(cfg, 21, 5)
    out = eng.step([("a", pa, [0, 15, 16, 44]), ("b", pb, [20])])
    assert eng.passes == 5
    wa, wb = Z.forward(cfg, st, pa), Z.forward(cfg, st, pb)
    assert rel(out[:4], wa[[0, 15, 16, 44]]) < 3e-6 and rel(out[4], wb[20]) < 3e-6


@pytest.mark.parametrize("kind", ["keyval", "diff", "diff_shared"])
def test_a_far_first_token_in_decoding(kind):
    """300 positions; two prompts that differ in their first token only must differ at the end, in
    the plain model and, decoded token by token over page borders, in the engine.  (Score scales
    chosen so that the first key keeps a share that shows: sharp maps for the differential layers,
    whose second map cancels what is spread evenly, flat ones beside the unit term.)"""
    layers = {"keyval": [keyval(heads=2, kv_heads=1, dim=8, rot=4, scale=0.2, mlp=None)],
              "diff": [diff(heads=2, kv_heads=1, dim=8, vdim=8, rot=4, scale=3.0, mlp=None)],
              "diff_shared": [diff(heads=2, kv_heads=1, dim=8, vdim=8, rot=4, scale=3.0, mlp=None),
                              diff(heads=2, kv_heads=1, dim=8, vdim=8, rot=4, scale=3.0, kv_from=0, mlp=None)]}[kind]
    cfg = model_cfg(layers)
    st = Z.random_tensors(cfg, 5)
    base, other = prompt(cfg, 300, 6), prompt(cfg, 300, 6)
    other[0] = (base[0] + 1) % cfg["vocab"]
    wa, wb = Z.forward(cfg, st, base), Z.forward(cfg, st, other)
    assert rel(wa[-1], wb[-1]) > 1e-4 and rel(wa[1], wb[1]) > 1e-3
    _, eng = build(cfg, st=st, max_seqs=2, max_tokens=1024)
    eng.step([("a", base[:100], [])])
    ga = torch.cat([eng.step([("a", [t], [0])]) for t in base[100:]])
    gb = eng.step([("b", other, [299])])
    assert rel(ga[-1], wa[-1]) < 3e-6 and rel(gb[0], wb[-1]) < 3e-6 and rel(ga, wa[100:]) < 3e-6
    eng.finish("b")
    g1 = eng.step([("c", other[:2], [0, 1])])            # the first tokens of a sequence
    assert rel(g1, wb[:2]) < 3e-6


def test_nothing_later_is_seen_at_page_borders():
    """A token changed at position p leaves every earlier position's logits as they were and moves
    position p's: at a page's last row, the next page's first row and around them, in a prompt cut
    there and in single decoded tokens."""
    cfg = SHAPES["two_kinds"]
    st = Z.random_tensors(cfg, 4)
    base = prompt(cfg, 40, 8)
    for p in (15, 16, 17, 31, 32):
        changed = list(base)
        changed[p] = (base[p] + 1) % cfg["vocab"]
        w0, w1 = Z.forward(cfg, st, base), Z.forward(cfg, st, changed)
        assert rel(w1[:p], w0[:p]) < 1e-12 and rel(w1[p], w0[p]) > 1e-3
        _, eng = build(cfg, st=st, max_seqs=2, max_tokens=256)
        head = eng.step([("x", changed[:p], list(range(p)))])
        tail = torch.cat([eng.step([("x", [t], [0])]) for t in changed[p:]])
        assert rel(head, w0[:p]) < 3e-6 and rel(tail, w1[p:]) < 3e-6, p
        whole = eng.step([("y", changed, list(range(40)))])
        assert rel(whole, w1) < 3e-6


def test_long_decoding():
    cfg = SHAPES["odd"]
    st, eng = build(cfg)
    toks = prompt(cfg, 230, 7)
    want = Z.forward(cfg, st, toks)
    eng.step([("a", toks[:10], [])])
    got = torch.cat([eng.step([("a", [t], [0])]) for t in toks[10:]])
    assert rel(got, want[10:]) < 5e-6
    assert rel(got[-1], want[-1]) < 5e-6


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_decode_steps_replayed_as_graphs(dtype):
    cfg = SHAPES["aligned"]
    st, plain = build(cfg, dtype, use_graph=False)
    _, graphed = build(cfg, dtype, use_graph=True)
    ps = [prompt(cfg, n, i) for i, n in enumerate((7, 19, 3))]
    for eng in (plain, graphed):
        eng.step([(str(i), p[:-1], []) for i, p in enumerate(ps)])
    nxt = [p[-1] for p in ps]
    for step in range(12):
        a = plain.step([(str(i), [t], [0]) for i, t in enumerate(nxt)])
        b = graphed.step([(str(i), [t], [0]) for i, t in enumerate(nxt)])
        assert torch.equal(a, b), step
        nxt = a.argmax(1).tolist()
    assert graphed.graph_replays >= 10


def test_greedy_generation_through_worker_and_scheduler():
    from vllm_omni_draft_amd import config, weights
    from vllm_omni_draft_amd.scheduler import SpecDecodeScheduler
    from vllm_omni_draft_amd.seq_engine import SeqWorker, SeqWorkerConfig
    cfg = SHAPES["two_kinds"]
    st = Z.random_tensors(cfg, 3)
    mc = config.zopupel_config(cfg, {k: tuple(v.shape) for k, v in st.items()})
    worker = SeqWorker(SeqWorkerConfig(weights.seq_from_state_dict(mc, st, DEV, torch.float32), max_num_seqs=3,
                                       max_model_len=128))
    worker.init_device()
    worker.load_model()
    sched = SpecDecodeScheduler.for_worker(worker)
    prompts = [prompt(cfg, n, i) for i, n in enumerate((5, 33, 1, 18, 64, 9, 2))]   # more requests than slots
    reqs = sched.generate(prompts, max_tokens=10)
    assert worker.engine.free_slots == 3
    for p, r in zip(prompts, reqs):
        assert len(r.output_token_ids) == 10 and r.finish_reason == "length"
        toks = list(p)
        for tok in r.output_token_ids:
            logits = Z.forward(cfg, st, toks)[-1]
            best = int(logits.argmax())
            if tok != best:                      # legitimate only at a near-tie of the plain model
                top = torch.topk(logits, 2).values
                assert (top[0] - top[1]) / logits.std() < 1e-4
                break
            toks.append(tok)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_replay_command_line(tmp_path, dtype):
    """bin/trace_run on a checkpoint folder: the class chosen by config.json, steps read from
    standard input (portions beside single tokens, requests ended and their pages used again by a
    pool that holds two requests at most), logits written per step."""
    import json
    import os
    import subprocess
    import sys
    import numpy as np
    from safetensors.torch import save_file
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cfg = SHAPES["two_kinds"]
    st = {k: v.to(torch.bfloat16).float() for k, v in Z.random_tensors(cfg, 6).items()}
    model, out = tmp_path / "model", tmp_path / "out"
    model.mkdir()
    (model / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in st.items()}, str(model / "model.safetensors"))
    pa, pb, pc = prompt(cfg, 70, 1), prompt(cfg, 50, 2), prompt(cfg, 64, 3)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": pa[:33], "want": [0, 32]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": pa[33:35], "want": [1]}, {"id": "b", "tokens": pb[:49], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "b", "tokens": pb[49:], "want": [0]}], "end": ["b"]},
             {"step": 3, "entries": [{"id": "a", "tokens": pa[35:], "want": [34]}, {"id": "c", "tokens": pc, "want": [63]}], "end": ["a", "c"]}]
    run = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", str(model), "--dtype", dtype,
                          "--out", str(out), "--max-tokens", "192"], input="".join(json.dumps(s) + "\n" for s in steps),
                         capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr[-2000:]
    assert [l for l in run.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2", "done 3"]
    wa, wb, wc = (Z.forward(cfg, st, p) for p in (pa, pb, pc))
    want = {0: wa[[0, 32]], 1: wa[[34]], 2: wb[[49]], 3: torch.stack([wa[69], wc[63]])}
    for n, w in want.items():
        got = torch.from_numpy(np.fromfile(str(out / f"{n}.f32"), dtype="<f4").reshape(w.shape[0], cfg["vocab"]).copy())
        assert rel(got, w) < (3e-6 if dtype == "float32" else 5e-2), n
