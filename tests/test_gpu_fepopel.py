"""The Fepopel decoder family on the GPU against the plain CPU restatement in oracle/fepopel.py:
every mechanism alone through its entry point, then whole models through the engine (prompts
whole, token by token, in portions, in mixed batches, over reused slots and pages) and through
the worker and scheduler.  Small random models of several shapes; where random weights would hide
a fault (one far key among many, a sink, a chunk's edge) the inputs are made so that it shows."""
import math

import pytest
import torch

from oracle import fepopel as P

pytestmark = pytest.mark.gpu

DEV = "cuda"
PAGE = 16


def dev(t, dtype=None):
    return t.to(dtype or t.dtype).contiguous().to(DEV)


def i32(x):
    return torch.tensor(x, dtype=torch.int32, device=DEV)


def rel(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return ((a - b).pow(2).mean().sqrt() / b.pow(2).mean().sqrt().clamp_min(1e-30)).item()


# ------------------------------------------------------------------ model shapes
def latent(heads=2, dim=8, rot_dim=4, vdim=12, kv_rank=16, scale=0.3, base=10000.0, mlp="default"):
    m = dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank, scale=scale,
             rot={"dims": rot_dim, "base": base})
    return {"type": "latent_attention", "mixer": m, "mlp": experts() if mlp == "default" else mlp}


def chunked(heads=4, kv_heads=2, dim=8, vdim=12, size=7, scale=0.4, softcap=3.0, mlp="default"):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale, softcap=softcap, mask={"size": size})
    return {"type": "attention", "mixer": m, "mlp": experts() if mlp == "default" else mlp}


def experts(n=4, top=2, ff=24, scale=1.7, shared=20):
    out = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": n, "top": top, "scale": scale}}
    if shared:
        out["shared"] = {"ff": shared}
    return out


def dense(ff=40):
    return {"kind": "dense", "ff": ff}


def model_cfg(layers, width=32, vocab=80, eps=1e-5, scale=3.0, loop=None):
    cfg = {"architecture": "Fepopel", "width": width, "vocab": vocab, "norm": {"eps": eps},
           "embedding": {"scale": scale}, "layers": layers}
    if loop:
        cfg["loop"] = dict(zip(("start", "stop", "times"), loop))
    return cfg


SHAPES = {
    "two_kinds": model_cfg([latent(mlp=dense()), chunked(), latent()], loop=(0, 2, 2)),
    # sizes that divide nothing; every pair of sizes that may coincide made different; the repeated span
    # in the middle, three times, with a chunked layer inside; a layer without feed-forward; experts
    # without a shared one; all experts chosen
    "odd": model_cfg([chunked(heads=6, kv_heads=3, dim=12, vdim=20, size=5, softcap=1.5, mlp=dense(36)),
                      latent(heads=3, dim=12, rot_dim=6, vdim=10, kv_rank=21, mlp=None),
                      chunked(heads=2, kv_heads=2, dim=20, vdim=4, size=33, mlp=experts(3, 3, 10, 0.6, 0)),
                      latent(heads=5, dim=6, rot_dim=10, vdim=14, kv_rank=9, base=500.0, mlp=experts(5, 3, 20, 1.0, 12))],
                     width=40, vocab=131, eps=1e-6, loop=(1, 3, 3)),
    # one head, a chunk of one token, one expert, a span that runs once, scales of one, no rotated part
    "ones": model_cfg([latent(heads=1, dim=4, rot_dim=2, vdim=6, kv_rank=8, mlp=experts(1, 1, 8, 1.0, 4)),
                       chunked(heads=1, kv_heads=1, dim=8, vdim=12, size=1, scale=1.0, mlp=None),
                       latent(heads=2, dim=4, rot_dim=0, vdim=6, kv_rank=8, scale=1.0, mlp=dense(8))],
                      width=24, vocab=50, scale=1.0, loop=(2, 3, 1)),
    # no repeated span at all; a chunk longer than any prompt here
    "plain": model_cfg([chunked(size=500, softcap=50.0, mlp=dense()), latent(mlp=experts(6, 1, 16, 2.0, 8))]),
    # widths that are multiples of 32: bfloat16 serving takes the tiled linear kernels and the matrix cores
    "aligned": model_cfg([latent(heads=4, dim=16, rot_dim=16, vdim=8, kv_rank=64, mlp=experts(8, 2, 32, 1.5, 64)),
                          chunked(heads=4, kv_heads=1, dim=16, vdim=16, size=24, mlp=dense(96)),
                          latent(heads=4, dim=16, rot_dim=16, vdim=8, kv_rank=64, mlp=experts(8, 2, 32, 1.5, 64))],
                         width=64, vocab=178, loop=(0, 1, 2)),
    # heads wider than a lane group, a latent wider than two tiles of value columns
    "wide": model_cfg([latent(heads=2, dim=24, rot_dim=8, vdim=40, kv_rank=136),
                       chunked(heads=2, kv_heads=1, dim=72, vdim=136, size=40)], width=48, vocab=64, loop=(0, 2, 2)),
}


def build(cfg, dtype=torch.float32, seed=0, tiled=True, st=None, **eng_kw):
    from vllm_omni_draft_amd import config, weights
    from vllm_omni_draft_amd.seq_engine import SeqEngine, SeqEngineConfig
    st = st or P.random_tensors(cfg, seed)
    mc = config.fepopel_config(cfg, {k: tuple(v.shape) for k, v in st.items()})
    w = weights.seq_from_state_dict(mc, st, DEV, dtype, tiled=tiled)
    kw = dict(max_seqs=4, max_tokens=1024)
    kw.update(eng_kw)
    return st, SeqEngine(w, SeqEngineConfig(**kw))


def prompt(cfg, n, seed=0):
    g = torch.Generator().manual_seed(1000 + seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


def oracle_logits(cfg, st, toks, layer_out=None):
    return P.forward(cfg, st, toks, layer_out)


def fill_cache(k, v, pages_of, G):
    """k [n, G*dk], v [n, G*dv] or None for one sequence in slot 0 -> caches, block table."""
    from vllm_omni_draft_amd import ops
    n = k.shape[0]
    dk = k.shape[1] // G
    n_pages = max(pages_of) + 1
    kc = torch.zeros(n_pages, G, PAGE, dk, dtype=k.dtype, device=DEV)
    vc = None
    if v is not None:
        vc = torch.zeros(n_pages, G, PAGE, v.shape[1] // G, dtype=k.dtype, device=DEV)
    bt = torch.zeros(2, len(pages_of), dtype=torch.int32, device=DEV)
    bt[0] = i32(pages_of)
    ops.cache_append(dev(k.float()), dev(v.float()) if v is not None else None, kc, vc, i32(list(range(n))),
                     i32([0] * n), bt, G, dk, v.shape[1] // G if v is not None else 0)
    return kc, vc, bt


# ------------------------------------------------------------------ mechanisms alone
@pytest.mark.parametrize("H,G,dk,dv,chunk,cap,sink", [(4, 2, 16, 16, 6, 2.0, False), (3, 1, 12, 20, 0, 0.0, True),
                                                      (2, 2, 72, 136, 1, 5.0, True), (9, 1, 8, 8, 17, 0.0, False),
                                                      (16, 2, 8, 300, 16, 0.7, True)])
@pytest.mark.parametrize("cdt", [torch.float32, torch.bfloat16])
def test_masked_softmax_attention_random(H, G, dk, dv, chunk, cap, sink, cdt):
    from vllm_omni_draft_amd import ops
    g = torch.Generator().manual_seed(H * 100 + dk)
    n = 45
    q = torch.randn(n, H * dk, generator=g)
    k, v = torch.randn(n, G * dk, generator=g).to(cdt), torch.randn(n, G * dv, generator=g).to(cdt)
    sinks = torch.randn(H, generator=g) * 2 if sink else None
    kc, vc, bt = fill_cache(k, v, [5, 1, 3], G)       # pages out of order
    rows = sorted({r for r in (0, 1, 2, chunk - 1, chunk, chunk + 1, 16, 31, 32, 44) if 0 <= r < n})
    want = P.attend(q[rows].view(-1, H, dk), k.view(n, G, dk), v.view(n, G, dv), rows, 0.2, chunk, cap, sinks)
    for split in (True, False):
        out = ops.masked_softmax_attention(dev(q[rows]), kc, vc, i32(rows), i32([0] * len(rows)), bt, H, G, dk, dv,
                                           0.2, chunk=chunk, softcap=cap, sinks=dev(sinks) if sink else None,
                                           split=split)
        assert rel(out, want.reshape(len(rows), -1)) < 3e-6


def test_a_sink_takes_its_share():
    """With keys that all score zero, a head's weights are 1 / (keys + exp(sink)) each: the output
    is the mean value times keys / (keys + exp(sink)); a very low sink changes nothing, a very high
    one leaves nothing; the first token of a sequence shares with the sink alone."""
    from vllm_omni_draft_amd import ops
    n, H, dk, dv = 40, 3, 8, 5
    g = torch.Generator().manual_seed(1)
    k, v = torch.zeros(n, dk), torch.randn(n, dv, generator=g)
    kc, vc, bt = fill_cache(k, v, [2, 0, 1], 1)
    sinks = torch.tensor([math.log(3.0), -80.0, 60.0])
    rows = [0, 1, 17, 39]
    q = torch.randn(len(rows), H * dk, generator=g)
    for each in (False, True):         # all rows in one launch, and one decoded row per launch
        if each:
            out = torch.cat([ops.masked_softmax_attention(dev(q[a:a + 1]), kc, vc, i32([r]), i32([0]), bt, H, 1, dk, dv,
                                                          1.0, sinks=dev(sinks)) for a, r in enumerate(rows)])
        else:
            out = ops.masked_softmax_attention(dev(q), kc, vc, i32(rows), i32([0] * len(rows)), bt, H, 1, dk, dv, 1.0,
                                               sinks=dev(sinks))
        out = out.view(len(rows), H, dv).cpu().double()
        for a, r in enumerate(rows):
            mean = v[:r + 1].double().mean(0)
            assert torch.allclose(out[a, 0], mean * (r + 1) / (r + 1 + 3.0), atol=1e-6)
            assert torch.allclose(out[a, 1], mean, atol=1e-6)
            assert out[a, 2].abs().max() < 1e-20


@pytest.mark.parametrize("chunk", [1, 2, 5, 16, 17, 32, 33, 300])
@pytest.mark.parametrize("decode", [False, True])
def test_masked_softmax_attention_sees_exactly_its_chunk(chunk, decode):
    """Key j carries a score far above all others only for the query that looks for j, and value
    one-hot(j): the output of query (i, target j) is one-hot(j) if i sees j, else has no weight on
    j.  Every (position, target) pair near a border: a chunk's first and last token, page borders,
    the sequence's first tokens."""
    from vllm_omni_draft_amd import ops
    n, dk = 70, 8
    dv = n
    gen = torch.Generator().manual_seed(chunk)
    code = torch.randn(n, dk, generator=gen)
    code = code / code.norm(dim=1, keepdim=True)
    kc, vc, bt = fill_cache(code.clone(), torch.eye(n), [4, 0, 2, 3, 1], 1)

    def targets(i):
        lo = i - i % chunk
        return sorted({j for j in (0, 1, lo - 2, lo - 1, lo, lo + 1, i - 1, i, 15, 16, 17, 31, 32) if 0 <= j <= i})
    pairs = [(i, j) for i in range(n) for j in targets(i)]
    if decode:      # one launch per query row, as single decoded tokens come
        keep = {0, 1, chunk - 1, chunk, chunk + 1, 2 * chunk - 1, 2 * chunk, 16, 33, n - 1}
        pairs = [p for p in pairs if p[0] in keep]
        out = torch.cat([ops.masked_softmax_attention(dev(code[j:j + 1] * 60), kc, vc, i32([i]), i32([0]), bt, 1, 1,
                                                      dk, dv, 1.0, chunk=chunk) for i, j in pairs]).cpu()
    else:
        q = torch.stack([code[j] * 60 for _, j in pairs])
        out = ops.masked_softmax_attention(dev(q), kc, vc, i32([i for i, _ in pairs]), i32([0] * len(pairs)), bt, 1, 1,
                                           dk, dv, 1.0, chunk=chunk).cpu()
    for r, (i, j) in enumerate(pairs):
        assert abs(out[r].sum().item() - 1) < 1e-4                  # a softmax: the weights sum to one
        assert torch.all(out[r, i + 1:] == 0), (i, j)               # nothing from the future
        assert torch.all(out[r, :i - i % chunk] == 0), (i, j)       # nothing from the chunks before
        if P.visible(i, j, chunk):
            assert out[r, j] > 0.5, (i, j, out[r, j].item())
        else:
            assert out[r, j] == 0, (i, j, out[r, j].item())


@pytest.mark.parametrize("cdt", [torch.float32, torch.bfloat16])
def test_masked_softmax_attention_many_keys_and_a_cap(cdt):
    """More keys than two tiles, no window: a far key that stands out in the first tile takes all
    the weight; with a cap its lead shrinks to what the cap allows."""
    from vllm_omni_draft_amd import ops
    g = torch.Generator().manual_seed(9)
    n, H, G, dk, dv = 700, 2, 1, 16, 24
    q = torch.randn(4, H * dk, generator=g)
    k, v = torch.randn(n, dk, generator=g).to(cdt), torch.randn(n, dv, generator=g).to(cdt)
    k[3] = (q[0, :dk] * 3).to(cdt)                     # row 699 of head 0 finds key 3
    sinks = torch.tensor([0.5, -1.0])
    kc, vc, bt = fill_cache(k, v, torch.randperm(44, generator=g).tolist(), G)
    rows = [699, 698, 650, 300]
    for cap in (0.0, 4.0):
        want = P.attend(q.view(4, H, dk), k.view(n, G, dk), v.view(n, G, dv), rows, 0.5, 0, cap, sinks)
        out = ops.masked_softmax_attention(dev(q), kc, vc, i32(rows), i32([0] * 4), bt, H, G, dk, dv, 0.5, softcap=cap,
                                           sinks=dev(sinks))
        whole = ops.masked_softmax_attention(dev(q), kc, vc, i32(rows), i32([0] * 4), bt, H, G, dk, dv, 0.5,
                                             softcap=cap, sinks=dev(sinks), split=False)
        assert rel(out, want.reshape(4, -1)) < 3e-6 and rel(whole, want.reshape(4, -1)) < 3e-6
        if cap == 0.0:
            assert rel(out[0, :dv], v[3].double()) < 1e-3
        else:
            assert rel(out[0, :dv], v[3].double()) > 0.1
    many = list(range(600, 700))
    q2 = torch.randn(100, H * dk, generator=g)
    out2 = ops.masked_softmax_attention(dev(q2), kc, vc, i32(many), i32([0] * 100), bt, H, G, dk, dv, 0.5, sinks=dev(sinks))
    one = ops.masked_softmax_attention(dev(q2[37:38]), kc, vc, i32(many[37:38]), i32([0]), bt, H, G, dk, dv, 0.5,
                                       sinks=dev(sinks))
    assert rel(one[0], out2[37]) < 2e-6


@pytest.mark.parametrize("H,G,dk,dv", [(4, 2, 16, 8), (5, 5, 12, 20), (1, 1, 130, 4), (12, 3, 8, 8)])
def test_heads_normed_one_by_one_and_appended(H, G, dk, dv):
    from vllm_omni_draft_amd import ops
    g = torch.Generator().manual_seed(H + dk)
    n, eps = 21, 1e-3
    q, k, v = torch.randn(n, H * dk, generator=g), torch.randn(n, G * dk, generator=g) * 3, torch.randn(n, G * dv, generator=g)
    qw, kw = 1 + torch.randn(dk, generator=g) * 0.2, 1 + torch.randn(dk, generator=g) * 0.2
    pages = [3, 0]
    kc = torch.zeros(4, G, PAGE, dk, device=DEV)
    vc = torch.zeros(4, G, PAGE, dv, device=DEV)
    bt = torch.zeros(1, 2, dtype=torch.int32, device=DEV)
    bt[0] = i32(pages)
    qd, kd = dev(q), dev(k)
    ops.qk_head_norm_append(qd, dev(qw), kd, dev(kw), dev(v), H, G, dk, dv, eps, kc, vc, i32(list(range(n))),
                            i32([0] * n), bt)
    wq = P.rms_norm(q.view(n, H, dk), qw, eps).reshape(n, -1)
    wk = P.rms_norm(k.view(n, G, dk), kw, eps)
    assert rel(qd, wq) < 2e-6 and rel(kd, wk.reshape(n, -1)) < 2e-6
    for t in (0, 15, 16, 20):
        pg = pages[t // PAGE]
        assert rel(kc[pg, :, t % PAGE], wk[t]) < 2e-6
        assert torch.equal(vc[pg, :, t % PAGE].cpu(), v[t].view(G, dv))


def test_latent_rows_without_a_query_latent():
    from vllm_omni_draft_amd import ops
    g = torch.Generator().manual_seed(2)
    n, rk, dr, eps, base = 19, 20, 6, 1e-5, 300.0
    kv = torch.randn(n, rk + dr, generator=g)
    w = 1 + torch.randn(rk, generator=g) * 0.1
    pos = list(range(5, 5 + n))
    kc = torch.zeros(3, 1, PAGE, rk + dr, device=DEV)
    bt = torch.zeros(1, 2, dtype=torch.int32, device=DEV)
    bt[0] = i32([2, 1])
    inv = torch.tensor(base, dtype=torch.float64) ** (-2.0 * torch.arange(dr // 2, dtype=torch.float64) / dr)
    kvd = dev(kv)
    ops.latent_kv_prep(kvd, dev(w), rk, dr, eps, dr, dev(inv), kc, i32(pos), i32([0] * n), bt)
    want = torch.cat([P.rms_norm(kv[:, :rk], w, eps), P.rotate_pairs(kv[:, rk:], torch.tensor(pos), dr, base)], 1)
    assert rel(kvd, want) < 2e-6
    assert rel(kc[1, 0, 0], want[pos.index(16)]) < 2e-6 and rel(kc[2, 0, 5], want[0]) < 2e-6


def test_head_gates_and_activations():
    from vllm_omni_draft_amd import ops
    g = torch.Generator().manual_seed(4)
    y, z = torch.randn(13, 5 * 12, generator=g), torch.randn(13, 5, generator=g) * 3
    yd = dev(y)
    ops.head_gate_rows(yd, dev(z), 5, 12)
    assert rel(yd, (y.double().view(13, 5, 12) * torch.sigmoid(z.double())[..., None]).reshape(13, -1)) < 1e-6
    a, b = torch.randn(9, 300, generator=g) * 2, torch.randn(9, 300, generator=g)
    ad, bd = a.double(), b.double()
    assert rel(ops.act_rows(dev(a), dev(b), "silu"), ad * torch.sigmoid(ad) * bd) < 1e-6
    assert rel(ops.act_rows(dev(a), dev(b), "relu"), torch.relu(ad) * bd) < 1e-6
    out, ob = ops.act_rows(dev(a), None, "relu2", bf16_copy=True)
    assert rel(out, torch.relu(ad).pow(2)) < 1e-2
    assert torch.equal(ob.float(), out)            # the bfloat16 copy holds the values the f32 rows were rounded to


@pytest.mark.parametrize("E,K,top,wdt", [(5, 40, 3, torch.float32), (16, 1000, 2, torch.bfloat16), (130, 64, 7, torch.float32),
                                         (1, 24, 1, torch.float32), (4, 32, 4, torch.float32)])
def test_router_with_scaled_weights_and_a_gate_row(E, K, top, wdt):
    from vllm_omni_draft_amd import ops
    g = torch.Generator().manual_seed(E)
    x = torch.randn(33, K, generator=g)
    w, wg = (torch.randn(E, K, generator=g) * 0.3).to(wdt), (torch.randn(2, K, generator=g) * 0.3).to(wdt)
    xr = x.bfloat16().float() if wdt == torch.bfloat16 else x
    sel_e, sel_w, logits, gates = ops.moe_route_rows_gated(dev(x), dev(w), top, "softmax", True, 1e-20, 1.7, dev(wg))
    idx, wt = P.route(xr, w.float(), top, 1.7)
    assert rel(logits, xr.double() @ w.double().T) < 2e-6
    assert rel(gates, xr.double() @ wg.double().T) < 2e-6
    assert torch.equal(sel_e.cpu().long(), idx)
    assert rel(sel_w, wt) < 2e-6
    assert torch.allclose(sel_w.sum(1).cpu(), torch.full((33,), 1.7), atol=1e-5)


@pytest.mark.parametrize("E,top,F,W,rows", [(4, 2, 24, 32, 9), (5, 3, 20, 40, 70), (1, 1, 8, 24, 3), (16, 1, 64, 48, 150),
                                            (8, 2, 64, 64, 5), (8, 2, 64, 64, 300), (8, 8, 32, 96, 40)])
@pytest.mark.parametrize("wdt", [torch.float32, torch.bfloat16])
def test_experts_of_two_matrices(E, top, F, W, rows, wdt):
    """down_e(relu(up_e x)^2) times the weight, for every chosen expert: few rows (a matrix-vector
    product each), many rows (grouped by expert), widths that take the matrix cores and widths that
    do not."""
    from vllm_omni_draft_amd import ops
    g = torch.Generator().manual_seed(E * 10 + top)
    x = torch.randn(rows, W, generator=g)
    up, down = (torch.randn(E, F, W, generator=g) * W ** -0.5).to(wdt), (torch.randn(E, W, F, generator=g) * F ** -0.5).to(wdt)
    sel_e = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(rows)]).int()
    sel_w = torch.rand(rows, top, generator=g) + 0.2
    out = ops.moe_experts(dev(x), dev(sel_e), dev(sel_w), dev(up), dev(down), scale_input=False, act="relu2")
    xr = x.bfloat16().float() if wdt == torch.bfloat16 else x
    want = torch.stack([torch.stack([sel_w[r, j].double() * P.squared_relu_ff(xr[r:r + 1], up[sel_e[r, j]].float(),
                                                                                 down[sel_e[r, j]].float())[0]
                                     for j in range(top)]) for r in range(rows)])
    assert rel(out, want) < (3e-6 if wdt == torch.float32 else 1e-2)


@pytest.mark.parametrize("W", [5, 72, 1000, 2048, 4100])
def test_residual_update_and_following_norm(W):
    from vllm_omni_draft_amd import ops
    g = torch.Generator().manual_seed(W)
    n, eps = 7, 1e-4
    x, a, b = torch.randn(n, W, generator=g), torch.randn(n * 3, W, generator=g), torch.randn(n, W, generator=g)
    gate, add = torch.randn(n, 1, generator=g), torch.randn(W, generator=g)
    wp, wn = 1 + torch.randn(W, generator=g) * 0.1, 1 + torch.randn(W, generator=g) * 0.1
    xd = dev(x)
    copy, h = ops.residual_norm(xd, dev(a), dev(wp), 3, dev(b), dev(gate), dev(add), dev(wn), eps, want_copy=True)
    t = a.double().view(n, 3, W).sum(1) + torch.sigmoid(gate.double()) * b.double()
    x1 = x.double() + P.rms_norm(t, wp, eps)
    assert rel(copy, x1) < 1e-6 and rel(xd, x1 + add.double()) < 1e-6
    assert rel(h, P.rms_norm(x1 + add.double(), wn, eps)) < 2e-6
    # nothing to add, only the norm of what is there (a model's first layer)
    x2 = dev(x)
    _, h2 = ops.residual_norm(x2, w_next=dev(wn), eps=eps)
    assert torch.equal(x2.cpu(), x) and rel(h2, P.rms_norm(x, wn, eps)) < 2e-6
    # one term, no gate, no following norm (a model's last layer)
    x3 = dev(x)
    ops.residual_norm(x3, dev(b), dev(wp), eps=eps)
    assert rel(x3, x.double() + P.rms_norm(b, wp, eps)) < 1e-6


# ------------------------------------------------------------------ whole models
@pytest.mark.parametrize("shape", list(SHAPES))
def test_prompt_logits_match_the_plain_model(shape):
    cfg = SHAPES[shape]
    st, eng = build(cfg)
    toks = prompt(cfg, 61)
    lo = []
    want = oracle_logits(cfg, st, toks, lo)
    got, trace = eng.step([("a", toks, list(range(len(toks))))], layer_out=True)
    assert trace.shape[0] == len(lo) == len(P.layer_runs(cfg))
    for i, x in enumerate(lo):
        assert rel(trace[i], x) < 3e-6, f"residual after layer run {i}"
    assert rel(got, want) < 3e-6


@pytest.mark.parametrize("shape,tiled", [("two_kinds", False), ("odd", False), ("aligned", True), ("aligned", False),
                                         ("wide", False)])
def test_bfloat16_serving_stays_close(shape, tiled):
    cfg = SHAPES[shape]
    st, eng = build(cfg, torch.bfloat16, tiled=tiled)
    toks = prompt(cfg, 50, 1)
    want = oracle_logits(cfg, st, toks)
    got = eng.step([("a", toks, list(range(len(toks))))])
    # (a token whose router scores lie within bfloat16 rounding of each other may take another
    # expert than the plain model, and the tokens behind it feel that: most rows are close)
    rows = sorted(rel(got[r], want[r]) for r in range(len(toks)))
    assert rows[len(rows) // 2] < 2e-2 and rows[int(len(rows) * 0.9)] < 6e-2, rows[-5:]


@pytest.mark.parametrize("shape,dtype,tiled", [("two_kinds", torch.float32, True), ("odd", torch.float32, True),
                                               ("ones", torch.float32, True), ("wide", torch.float32, True),
                                               ("plain", torch.float32, True),
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
            assert rel(whole[name], oracle_logits(cfg, st, p)) < 3e-6

    def same(x, y, what):
        # (few rows cut their keys over workgroups and merge them, many rows sweep them in one:
        # the two orders of summation differ in the last bits)
        assert rel(x, y) < (1e-5 if dtype == torch.float32 else 1e-2), what
    # token by token
    eng.step([("pad", prompt(cfg, 20, 9), [])])       # another slot and other pages than before
    got = torch.cat([eng.step([("a", [t], [0])]) for t in pa])
    same(got, whole["a"], "token by token")
    eng.finish("a")
    # portions of changing size, down to two tokens, beside other requests' portions and single tokens
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
        ref[r] = (p, oracle_logits(cfg, st, p)[-1])
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


def test_a_step_larger_than_a_pass():
    cfg = SHAPES["two_kinds"]
    st, eng = build(cfg, max_rows=16)
    pa, pb = prompt(cfg, 45, 4), prompt(cfg, 21, 5)
    out = eng.step([("a", pa, [0, 15, 16, 44]), ("b", pb, [20])])
    assert eng.passes == 5
    wa, wb = oracle_logits(cfg, st, pa), oracle_logits(cfg, st, pb)
    assert rel(out[:4], wa[[0, 15, 16, 44]]) < 3e-6 and rel(out[4], wb[20]) < 3e-6


def test_a_far_token_through_latent_attention():
    """One latent-attention layer whose last position looks for the first token among hundreds:
    queries and keys are scaled up so that the first token's key stands out, and only the first
    token differs between two prompts.  The engine, decoding token by token, must still feel it."""
    cfg = model_cfg([latent(heads=2, dim=8, rot_dim=0, vdim=8, kv_rank=16, scale=1.0, mlp=None)])
    st = P.random_tensors(cfg, 5)
    st["l0.mix.sink"] = torch.tensor([-30.0, -30.0])
    base, other = prompt(cfg, 300, 6), prompt(cfg, 300, 6)
    other[0] = (base[0] + 1) % cfg["vocab"]
    wa, wb = oracle_logits(cfg, st, base), oracle_logits(cfg, st, other)
    _, eng = build(cfg, st=st, max_seqs=2, max_tokens=1024)
    eng.step([("a", base[:100], [])])
    ga = torch.cat([eng.step([("a", [t], [0])]) for t in base[100:]])
    gb = eng.step([("b", other, [299])])
    assert rel(ga[-1], wa[-1]) < 3e-6 and rel(gb[0], wb[-1]) < 3e-6
    # the position just behind the first token attends to two keys only: there the difference is large
    assert rel(wa[1], wb[1]) > 1e-3
    eng.finish("b")
    g1 = eng.step([("c", other[:2], [1])])
    assert rel(g1[0], wb[1]) < 3e-6


def test_a_chunk_edge_in_prompts_and_in_decoding():
    """One chunked layer, queries and keys scaled so that attention is sharp: the logits at a
    chunk's first position must not depend on the token just before it, those at a chunk's last
    position must depend on the chunk's first token; both for positions inside a prompt portion
    and for single decoded tokens."""
    size = 9
    cfg = model_cfg([chunked(heads=2, kv_heads=1, dim=8, vdim=8, size=size, scale=1.0, softcap=30.0, mlp=None)])
    st = P.random_tensors(cfg, 8)
    base = prompt(cfg, 40, 3)
    first, last = 2 * size, 3 * size - 1           # a chunk's first and last position
    out_tok = list(base)
    out_tok[first - 1] = (base[first - 1] + 1) % cfg["vocab"]      # just outside the chunk of `first`
    in_tok = list(base)
    in_tok[first] = (base[first] + 1) % cfg["vocab"]               # the first token of the chunk of `last`
    w0, w_out, w_in = (oracle_logits(cfg, st, t) for t in (base, out_tok, in_tok))
    assert rel(w_out[first], w0[first]) < 1e-12 and rel(w_in[last], w0[last]) > 1e-4
    for cut in (None, first - 1, first, first + 1):
        _, eng = build(cfg, st=st, max_seqs=2, max_tokens=256)
        for name, toks, want in (("o", out_tok, w_out), ("i", in_tok, w_in)):
            if cut is None:
                got = eng.step([(name, toks, [first, last])])
            else:      # a prompt portion up to `cut`, the rest token by token
                head = eng.step([(name, toks[:cut], [first] if first < cut else [])])
                rows = torch.cat([eng.step([(name, [t], [0])]) for t in toks[cut:]])
                got = torch.stack([head[0] if first < cut else rows[first - cut], rows[last - cut]])
            assert rel(got[0], want[first]) < 3e-6 and rel(got[1], want[last]) < 3e-6, (cut, name)


def test_long_decoding():
    cfg = SHAPES["odd"]
    st, eng = build(cfg)
    toks = prompt(cfg, 230, 7)
    want = oracle_logits(cfg, st, toks)
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
    st = P.random_tensors(cfg, 3)
    mc = config.fepopel_config(cfg, {k: tuple(v.shape) for k, v in st.items()})
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
            logits = oracle_logits(cfg, st, toks)[-1]
            best = int(logits.argmax())
            if tok != best:                      # legitimate only at a near-tie of the plain model
                top = torch.topk(logits, 2).values
                assert (top[0] - top[1]) / logits.std() < 1e-4
                break
            toks.append(tok)
