"""Host-side parts of the Fepopel family that need no GPU: the configuration reader and model
registry, the order in which repeated layers run, the caches' shapes (one per run), the stacked
weights, and the plain CPU model's own consistency (causality, the chunk rule, the sink, the
absorbed form of latent attention, routing)."""
import json
import math
import os
import subprocess

import pytest
import torch

from oracle import fepopel as P

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

MOE = {"kind": "moe", "expert": {"ff": 20}, "router": {"experts": 5, "top": 2, "scale": 1.3}, "shared": {"ff": 12}}
CFG = {"architecture": "Fepopel", "width": 40, "vocab": 70, "norm": {"eps": 1e-6}, "embedding": {"scale": 5.0},
       "loop": {"start": 1, "stop": 3, "times": 2},
       "layers": [
           {"type": "latent_attention", "mlp": {"kind": "dense", "ff": 28},
            "mixer": {"heads": 3, "dim": 8, "rot_dim": 4, "vdim": 12, "kv_rank": 14, "scale": 0.4,
                      "rot": {"dims": 4, "base": 500.0}}},
           {"type": "attention", "mlp": None,
            "mixer": {"heads": 4, "kv_heads": 2, "dim": 8, "vdim": 6, "scale": 0.5, "softcap": 2.5, "mask": {"size": 5}}},
           {"type": "latent_attention", "mlp": MOE,
            "mixer": {"heads": 2, "dim": 6, "rot_dim": 2, "vdim": 10, "kv_rank": 9, "scale": 0.7,
                      "rot": {"dims": 2, "base": 10000.0}}},
       ]}


def test_chunk_rule():
    for chunk in (0, 1, 2, 5):
        for i in range(20):
            seen = [j for j in range(25) if P.visible(i, j, chunk)]
            lo = 0 if chunk == 0 else i - i % chunk
            assert seen == list(range(lo, i + 1))
        # the attention of the plain model applies the same rule: one-hot values show who is seen
        q, k, v = torch.zeros(20, 1, 2, dtype=torch.float64), torch.zeros(25, 1, 2, dtype=torch.float64), torch.eye(25, dtype=torch.float64)[:, None, :]
        w = P.attend(q, k, v, list(range(20)), 1.0, chunk=chunk)[:, 0]
        for i in range(20):
            assert [j for j in range(25) if w[i, j] > 0] == [j for j in range(25) if P.visible(i, j, chunk)]


def test_order_of_running():
    assert P.layer_runs(CFG) == [(0, None), (1, 0), (2, 0), (1, 1), (2, 1)]
    assert P.layer_runs({"layers": [0, 0]}) == [(0, None), (1, None)]
    cfg = dict(CFG, loop={"start": 0, "stop": 3, "times": 3})
    assert [i for i, _ in P.layer_runs(cfg)] == [0, 1, 2] * 3


def test_plain_model_is_causal_and_chunks_count_from_the_start():
    st = P.random_tensors(CFG, 1)
    g = torch.Generator().manual_seed(0)
    toks = torch.randint(0, CFG["vocab"], (40,), generator=g).tolist()
    whole = P.forward(CFG, st, toks)
    for n in (1, 5, 6, 23):
        assert torch.allclose(P.forward(CFG, st, toks[:n]), whole[:n], atol=1e-10, rtol=0)
    # a prompt that starts one token later is another sequence: its chunks lie elsewhere
    assert not torch.allclose(P.forward(CFG, st, toks[1:])[-1], whole[-1], atol=1e-6)


def test_sink_is_one_more_term_of_the_denominator():
    g = torch.Generator().manual_seed(3)
    q, k, v = (torch.randn(6, 2, 4, generator=g, dtype=torch.float64) for _ in range(3))
    sink = torch.tensor([0.3, -1.2], dtype=torch.float64)
    out = P.attend(q, k, v, list(range(6)), 0.5, sink=sink)
    for i in range(6):
        for h in range(2):
            s = torch.tensor([float(q[i, h] @ k[j, h]) * 0.5 for j in range(i + 1)], dtype=torch.float64)
            w = torch.exp(s) / (torch.exp(s).sum() + math.exp(float(sink[h])))
            assert torch.allclose(out[i, h], (w[:, None] * v[:i + 1, h]).sum(0), atol=1e-12)
    # a very low sink is no sink
    plain = P.attend(q, k, v, list(range(6)), 0.5)
    assert torch.allclose(P.attend(q, k, v, list(range(6)), 0.5, sink=sink - 200), plain, atol=1e-12)


def test_capped_scores_and_grouped_heads():
    g = torch.Generator().manual_seed(4)
    q = torch.randn(5, 4, 3, generator=g, dtype=torch.float64) * 4
    k, v = (torch.randn(5, 2, 3, generator=g, dtype=torch.float64) for _ in range(2))
    out = P.attend(q, k, v, list(range(5)), 1.0, chunk=3, softcap=2.0)
    i, h = 4, 3                                    # position 4 sees 3 and 4; head 3 reads key head 1
    s = torch.stack([2.0 * torch.tanh(q[i, h] @ k[j, 1] / 2.0) for j in (3, 4)])
    w = torch.softmax(s, 0)
    assert torch.allclose(out[i, h], w[0] * v[3, 1] + w[1] * v[4, 1], atol=1e-12)


def test_latent_attention_equals_its_absorbed_form():
    """Scores and values can be taken against the cached latent itself: q' = U_k^T q per head,
    and the weighted latent expanded afterwards.  The plain model uses the expanded form."""
    m = dict(CFG["layers"][0]["mixer"], eps=1e-6)
    t = P.sub(P.random_tensors(CFG, 2), "l0.mix.")
    g = torch.Generator().manual_seed(1)
    T, H, dk, dr, dv, rk = 11, m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    h = torch.randn(T, CFG["width"], generator=g, dtype=torch.float64)
    pos = torch.arange(T)
    want = P.latent_attention(h, m, t, pos)
    q = (h @ t["q"].double().T).view(T, H, dk + dr)
    low = h @ t["dkv"].double().T
    row = torch.cat([P.rms_norm(low[:, :rk], t["dkv.norm"], 1e-6), P.rotate_pairs(low[:, rk:], pos, dr, 500.0)], 1)
    uk, uv = t["uk"].double().view(H, dk, rk), t["uv"].double().view(H, dv, rk)
    qe = torch.cat([torch.einsum("thd,hdr->thr", q[..., :dk], uk), P.rotate_pairs(q[..., dk:], pos, dr, 500.0)], -1)
    o = P.attend(qe, row[:, None, :], row[:, None, :rk], pos, m["scale"], sink=t["sink"])       # one shared key head
    y = torch.einsum("thr,hvr->thv", o, uv) * torch.sigmoid(h @ t["g"].double().T)[..., None]
    assert torch.allclose(y.reshape(T, -1) @ t["o"].double().T, want, atol=1e-10)


def test_routing_takes_the_largest_scores_and_scales_the_output():
    g = torch.Generator().manual_seed(4)
    t = {"router": torch.randn(5, 8, generator=g, dtype=torch.float64)}
    for e in range(5):
        t[f"e{e}.up"], t[f"e{e}.down"] = torch.randn(6, 8, generator=g, dtype=torch.float64), torch.randn(8, 6, generator=g, dtype=torch.float64)
    t["shared.up"], t["shared.down"] = torch.randn(4, 8, generator=g, dtype=torch.float64), torch.randn(8, 4, generator=g, dtype=torch.float64)
    t["shared.sg"] = torch.randn(1, 8, generator=g, dtype=torch.float64)
    h = torch.randn(3, 8, generator=g, dtype=torch.float64)
    mlp = {"router": {"experts": 5, "top": 2, "scale": 1.3}, "shared": {"ff": 4}}
    out = P.experts_ff(h, mlp, t)
    s = torch.softmax(h @ t["router"].T, -1)
    for r in range(3):
        best = sorted(range(5), key=lambda e: -s[r, e])[:2]
        tot = sum(s[r, e] for e in best)
        want = sum(1.3 * s[r, e] / tot * (t[f"e{e}.down"] @ torch.relu(t[f"e{e}.up"] @ h[r]) ** 2) for e in best)
        want = want + torch.sigmoid(t["shared.sg"][0] @ h[r]) * (t["shared.down"] @ torch.relu(t["shared.up"] @ h[r]) ** 2)
        assert torch.allclose(out[r], want, atol=1e-12)
    idx, wt = P.route(h, t["router"], 5, 0.5)
    assert torch.allclose(wt.sum(1), torch.full((3,), 0.5, dtype=torch.float64))
    assert torch.allclose(wt, 0.5 * s.gather(1, idx))         # all experts chosen: the scores themselves


def test_config_reader_and_registry(tmp_path):
    from safetensors.torch import save_file
    from vllm_omni_draft_amd import config
    st = P.random_tensors(CFG, 2)
    (tmp_path / "config.json").write_text(json.dumps(CFG))
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in st.items()}, str(tmp_path / "model.safetensors"))
    mc = config.load_model_config(str(tmp_path))
    assert isinstance(mc, config.SeqModelConfig) and (mc.arch, mc.block, mc.n_layers) == ("fepopel", "sandwich", 3)
    assert (mc.embed_scale, mc.logit_scale, mc.tied_head, mc.norm_eps, mc.bigram) == (5.0, 1.0, False, 1e-6, None)
    assert mc.loop == {"start": 1, "stop": 3, "times": 2} and mc.n_runs == 5
    assert mc.runs == P.layer_runs(CFG)
    a, b, c = (l.mixer for l in mc.layers)
    assert (a.kind, a.heads, a.dim, a.rot_dim, a.vdim, a.q_rank, a.kv_rank, a.window, a.rot_dims, a.rot_base) == \
        ("latent_attention", 3, 8, 4, 12, 0, 14, 0, 4, 500.0)
    assert a.rot_layout == "interleaved" and a.sink and a.head_gate and a.scale == 0.4
    assert (b.kind, b.heads, b.kv_heads, b.dim, b.vdim, b.chunk, b.softcap, b.scale, b.rot_dims, b.qk_head_norm) == \
        ("softmax_attention", 4, 2, 8, 6, 5, 2.5, 0.5, 0, True)
    assert (mc.layers[0].ff, mc.layers[0].ff_act, mc.layers[0].experts) == (28, "silu", None)
    assert mc.layers[1].ff == 0 and mc.layers[1].experts is None
    e = mc.layers[2].experts
    assert (e.experts, e.top, e.ff, e.score, e.renorm, e.scale_input, e.act, e.scale, e.renorm_eps, e.shared_ff) == \
        (5, 2, 20, "softmax", True, False, "relu2", 1.3, 1e-20, 12)
    assert mc.state_bytes_per_seq() == 0
    assert mc.param_count() == sum(v.numel() for v in st.values())
    # no repeated span, no shared expert
    cfg = json.loads(json.dumps(CFG))
    del cfg["loop"], cfg["layers"][2]["mlp"]["shared"]
    mc = config.fepopel_config(cfg)
    assert mc.loop is None and mc.runs == [(0, None), (1, None), (2, None)] and mc.layers[2].experts.shared_ff == 0


@pytest.mark.parametrize("path,value", [
    (("layers", 0, "type"), "conv"),
    (("layers", 0, "mixer", "rot", "dims"), 6),                 # more than the rotated channels
    (("layers", 0, "mixer", "rot", "dims"), 3),
    (("layers", 0, "mixer", "kv_rank"), 0),
    (("layers", 1, "mixer", "kv_heads"), 3),
    (("layers", 1, "mixer", "mask", "size"), -1),
    (("layers", 1, "mixer", "softcap"), -1.0),
    (("layers", 2, "mlp", "router", "top"), 6),
    (("layers", 2, "mlp", "kind"), "conv"),
    (("loop", "stop"), 4),
    (("loop", "start"), 3),
    (("loop", "times"), 0),
])
def test_config_reader_refuses(path, value):
    from vllm_omni_draft_amd import config
    cfg = json.loads(json.dumps(CFG))
    node = cfg
    for k in path[:-1]:
        node = node[k]
    node[path[-1]] = value
    with pytest.raises(ValueError):
        config.fepopel_config(cfg)


def test_every_run_of_a_layer_has_a_cache_of_its_own():
    from vllm_omni_draft_amd import _lib, config
    from vllm_omni_draft_amd.kv_cache import PAGE, SeqCache
    if not os.path.exists(_lib.lib_path()):
        subprocess.run(["make", "-C", ROOT, "-j8"], check=True)
    mc = config.fepopel_config(CFG)
    c = SeqCache(mc, torch.bfloat16, max_seqs=3, num_pages=7, max_seq_len=4 * PAGE, device="cpu")
    assert c.has_pages and sorted(c.k) == [0, 1, 2, 3, 4] and sorted(c.v) == [1, 3] and not c.state
    assert c.k[0].shape == (7, 1, PAGE, 14 + 4)              # one latent row per token, no values
    for run in (1, 3):                                       # layer 1 in both passes
        assert c.k[run].shape == (7, 2, PAGE, 8) and c.v[run].shape == (7, 2, PAGE, 6)
    for run in (2, 4):
        assert c.k[run].shape == (7, 1, PAGE, 9 + 2)
    assert c.k[1].data_ptr() != c.k[3].data_ptr() and c.k[0].dtype == torch.bfloat16


def test_weights_are_stacked_per_layer():
    from vllm_omni_draft_amd import config, weights
    st = P.random_tensors(CFG, 3)
    mc = config.fepopel_config(CFG)
    w = weights.seq_from_state_dict(mc, st, "cpu", torch.float32)
    a, b, c = w.layers
    assert a.w_in.shape == (3 * (8 + 4) + 14 + 4 + 3, 40)     # q | dkv | head gates
    assert torch.equal(a.w_in[-3:], st["l0.mix.g"]) and a.sinks.dtype == torch.float32
    assert a.w_uk_t.shape == (3, 14, 8) and torch.equal(a.w_uk_t[1].T, st["l0.mix.uk"][8:16])
    assert a.w_ff_in.shape == (56, 40) and torch.equal(a.w_ff_in[28:], st["l0.mlp.up"])
    assert b.w_in.shape == (4 * 8 + 2 * 8 + 2 * 6, 40) and b.q_norm_w.shape == (8,) and b.norm2_w is None
    assert c.w_gate_up.shape == (5, 20, 40) and c.w_down_e.shape == (5, 40, 20)
    assert c.w_shared_in.shape == (12, 40) and c.w_shared_gate.shape == (1, 40)
    assert w.loop_step.shape == (2, 40) and w.head.shape == (70, 40) and w.head_tiled is None
    st2 = weights.seq_random_state(mc, 0)
    assert {k: tuple(v.shape) for k, v in st2.items()} == {k: tuple(v.shape) for k, v in st.items()}
    del st["l2.mlp.shared.sg"]
    with pytest.raises(KeyError):
        weights.seq_from_state_dict(mc, st, "cpu", torch.float32)
