"""Host-side parts of the Zopupel family that need no GPU: the configuration reader and model
registry, the caches' shapes (several key rows per kv head, layers that own none), the stacked
weights, and the plain CPU model's own consistency (causality, the two score maps, the unit term
of the denominator, values taken from keys, shared keys, the rotary frequencies, routing)."""
import json
import math
import os
import subprocess

import pytest
import torch

from oracle import zopupel as Z

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
F64 = torch.float64

MOE = {"kind": "moe", "expert": {"ff": 20}, "router": {"experts": 5, "top": 2}, "shared": {"ff": 12}}
BLEND = {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}
CFG = {"architecture": "Zopupel", "width": 40, "vocab": 70, "norm": {"eps": 1e-6}, "residual_mult": 0.6,
       "layers": [
           {"type": "attention", "mlp": MOE,
            "mixer": {"heads": 4, "kv_heads": 2, "dim": 6, "vdim": 10, "scale": 0.4, "diff": 0.25,
                      "rot": {"dims": 4, "base": 500.0, "scaling": {"factor": 3.0}}}},
           {"type": "attention_2", "mlp": None,
            "mixer": {"heads": 3, "kv_heads": 1, "dim": 8, "vdim": 8, "scale": 0.5,
                      "rot": {"dims": 6, "base": 10000.0, "scaling": BLEND}}},
           {"type": "attention", "mlp": {"kind": "moe", "expert": {"ff": 9}, "router": {"experts": 3, "top": 3}},
            "mixer": {"heads": 4, "kv_heads": 2, "dim": 6, "vdim": 10, "scale": 0.4, "diff": 0.25, "kv_from": 0,
                      "rot": {"dims": 4, "base": 500.0, "scaling": {"factor": 3.0}}}},
       ]}


def toks(n, seed=0):
    return torch.randint(0, CFG["vocab"], (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def test_plain_model_is_causal():
    st = Z.random_tensors(CFG, 1)
    t = toks(40)
    whole = Z.forward(CFG, st, t)
    for n in (1, 5, 6, 23):
        assert torch.allclose(Z.forward(CFG, st, t[:n]), whole[:n], atol=1e-10, rtol=0)
    assert not torch.allclose(Z.forward(CFG, st, t[1:])[-1], whole[-1], atol=1e-6)     # positions count from 0


def test_unit_term_of_the_denominator():
    g = torch.Generator().manual_seed(3)
    s = torch.randn(2, 6, 6, generator=g, dtype=F64)
    w = Z.causal_softmax(s, list(range(6)), extra_one=True)
    for h in range(2):
        for i in range(6):
            e = torch.exp(s[h, i, :i + 1])
            assert torch.allclose(w[h, i, :i + 1], e / (1 + e.sum()), atol=1e-14) and w[h, i, i + 1:].abs().sum() == 0
    # very low scores: nearly all the weight goes to the term without a value; very high ones: nearly none
    assert Z.causal_softmax(s - 50, list(range(6)), extra_one=True).sum(-1).max() < 1e-18
    assert (Z.causal_softmax(s + 50, list(range(6)), extra_one=True).sum(-1) - 1).abs().max() < 1e-15
    assert torch.allclose(Z.causal_softmax(s, list(range(6))).sum(-1), torch.ones(2, 6, dtype=F64))


def test_two_maps_of_a_head_and_the_layer_number():
    m = dict(CFG["layers"][0]["mixer"], eps=1e-6)
    t = Z.sub(Z.random_tensors(CFG, 2), "l0.mix.")
    g = torch.Generator().manual_seed(1)
    T, H, G, dk, dv = 9, 4, 2, 6, 10
    h = torch.randn(T, CFG["width"], generator=g, dtype=F64)
    pos = torch.arange(T)
    want = Z.diff_attention(h, m, t, pos)
    lam = math.exp(float((t["lq1"] * t["lk1"]).sum())) - math.exp(float((t["lq2"] * t["lk2"]).sum())) + 0.25
    assert abs(Z.diff_lambda(t, 0.25) - lam) < 1e-6
    q = Z.rotate_half((h @ t["q"].double().T).view(T, H * 2, dk), pos, m["rot"]).view(T, H, 2, dk)
    k = Z.rotate_half((h @ t["k"].double().T).view(T, G * 2, dk), pos, m["rot"]).view(T, G, 2, dk)
    v = (h @ t["v"].double().T).view(T, G, dv)
    heads = []
    for hd in range(H):
        gk = hd // (H // G)
        maps = []
        for mp in range(2):
            rows = []
            for i in range(T):
                s = torch.stack([q[i, hd, mp] @ k[j, gk, mp] * 0.4 for j in range(i + 1)])
                rows.append(torch.softmax(s, 0) @ v[:i + 1, gk])
            maps.append(torch.stack(rows))
        o = maps[0] - Z.diff_lambda(t, 0.25) * maps[1]
        heads.append(o / torch.sqrt(o.pow(2).mean(-1, keepdim=True) + 1e-6) * 0.75)
    assert torch.allclose(torch.cat(heads, 1) @ t["o"].double().T, want, atol=1e-10)


def test_values_are_the_keys_as_projected():
    m = dict(CFG["layers"][1]["mixer"], eps=1e-6)
    t = Z.sub(Z.random_tensors(CFG, 2), "l1.mix.")
    g = torch.Generator().manual_seed(5)
    T = 7
    h = torch.randn(T, CFG["width"], generator=g, dtype=F64)
    want = Z.keyvalue_attention(h, m, t, torch.arange(T))
    # position 0 sees itself only: weight e^s / (1 + e^s) on its own value, the key before norm and turn
    q0 = Z.rms_norm(h[0] @ t["q"].double().T + t["q.b"].double(), t["q.norm"], 1e-6).view(3, 8)
    raw = h[0] @ t["k"].double().T + t["k.b"].double()
    k0 = Z.rms_norm(raw, t["k.norm"], 1e-6)
    mag = 0.1 * math.log(4.0) + 1.0
    grow = torch.tensor([mag] * 6 + [1.0] * 2, dtype=F64)      # position 0: no turn, but cos is multiplied by the factor
    out = []
    for hd in range(3):
        s = math.exp(float((q0[hd] * grow) @ (k0 * grow)) * 0.5)
        out.append(s / (1 + s) * raw)
    assert torch.allclose(torch.cat(out) @ t["o"].double().T + t["o.b"].double(), want[0], atol=1e-10)
    # the factor of cos and sin shows: it is not one here
    assert Z.frequencies(m["rot"])[1] == 0.1 * math.log(4.0) + 1.0


def test_shared_keys_equal_the_source_layers():
    """A layer that reads another layer's keys and values gives what its own projections would, if
    they were the source's and its input the source's input."""
    st = Z.random_tensors(CFG, 3)
    m0, m2 = dict(CFG["layers"][0]["mixer"], eps=1e-6), dict(CFG["layers"][2]["mixer"], eps=1e-6)
    g = torch.Generator().manual_seed(2)
    h0, h2 = (torch.randn(8, CFG["width"], generator=g, dtype=F64) for _ in range(2))
    pos = torch.arange(8)
    kv = Z.diff_keys_values(h0, m0, Z.sub(st, "l0.mix."), pos)
    t2 = Z.sub(st, "l2.mix.")
    assert "k" not in t2 and "v" not in t2
    got = Z.diff_attention(h2, m2, t2, pos, kv=kv)
    t_own = dict(t2, k=st["l0.mix.k"], v=st["l0.mix.v"])
    q_part = Z.diff_attention(h2, m2, t_own, pos, kv=Z.diff_keys_values(h0, m2, t_own, pos))
    assert torch.allclose(got, q_part, atol=1e-12)
    assert not torch.allclose(got, Z.diff_attention(h2, m2, t_own, pos), atol=1e-3)      # keys from its own input differ


def test_routing_is_a_softmax_over_the_chosen_logits():
    g = torch.Generator().manual_seed(4)
    t = {"router": torch.randn(5, 8, generator=g, dtype=F64), "router.b": torch.randn(5, generator=g, dtype=F64) * 2}
    for e in ["e%d" % i for i in range(5)] + ["shared"]:
        t[e + ".gate"], t[e + ".up"] = torch.randn(6, 8, generator=g, dtype=F64), torch.randn(6, 8, generator=g, dtype=F64)
        t[e + ".down"] = torch.randn(8, 6, generator=g, dtype=F64)
    h = torch.randn(3, 8, generator=g, dtype=F64)
    out = Z.experts_ff(h, {"router": {"experts": 5, "top": 2}, "shared": {"ff": 6}}, t)
    z = h @ t["router"].T + t["router.b"]

    def ff(e, x):
        a = t[e + ".gate"] @ x
        return t[e + ".down"] @ (a * torch.sigmoid(a) * (t[e + ".up"] @ x))

    for r in range(3):
        best = sorted(range(5), key=lambda e: -z[r, e])[:2]
        w = torch.softmax(torch.stack([z[r, e] for e in best]), 0)
        want = sum(w[i] * ff("e%d" % e, h[r]) for i, e in enumerate(best)) + ff("shared", h[r])
        assert torch.allclose(out[r], want, atol=1e-12)
    # the same weights as a softmax over all experts, renormed over the chosen ones
    idx, wt = Z.route(h, t["router"], t["router.b"], 2)
    p = torch.softmax(z, -1).gather(1, idx)
    assert torch.allclose(wt, p / p.sum(-1, keepdim=True), atol=1e-14)
    assert (Z.route(h, t["router"], torch.zeros(5, dtype=F64), 2)[0] != idx).any()       # the bias decides


def test_config_reader_and_registry(tmp_path):
    from safetensors.torch import save_file
    from vllm_omni_draft_amd import config
    st = Z.random_tensors(CFG, 2)
    (tmp_path / "config.json").write_text(json.dumps(CFG))
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in st.items()}, str(tmp_path / "model.safetensors"))
    mc = config.load_model_config(str(tmp_path))
    assert isinstance(mc, config.SeqModelConfig) and (mc.arch, mc.block, mc.n_layers) == ("zopupel", "sandwich", 3)
    assert (mc.residual_mult, mc.embed_scale, mc.tied_head, mc.norm_eps, mc.loop, mc.n_runs) == (0.6, 1.0, False, 1e-6, None, 3)
    a, b, c = (l.mixer for l in mc.layers)
    assert (a.kind, a.heads, a.kv_heads, a.dim, a.vdim, a.maps, a.diff, a.kv_from, a.window, a.chunk) == \
        ("softmax_attention", 4, 2, 6, 10, 2, 0.25, -1, 0, 0)
    assert (a.rot_dims, a.rot_base, a.rot_layout, a.rot_scaling) == (4, 500.0, "half", {"factor": 3.0})
    assert not (a.qk_head_norm or a.qk_full_norm or a.proj_bias or a.value_is_key or a.unit_sink or a.sink)
    assert (b.maps, b.qk_full_norm, b.proj_bias, b.value_is_key, b.unit_sink, b.rot_scaling) == (1, True, True, True, True, BLEND)
    assert c.kv_from == 0 and c.maps == 2
    e = mc.layers[0].experts
    assert (e.experts, e.top, e.ff, e.score, e.renorm, e.scale_input, e.act, e.shared_ff, e.shared_gate, e.router_bias) == \
        (5, 2, 20, "softmax", True, False, "silu", 12, False, True)
    assert mc.layers[1].experts is None and mc.layers[2].experts.shared_ff == 0
    assert mc.state_bytes_per_seq() == 0
    assert mc.param_count() == sum(v.numel() for v in st.values())


@pytest.mark.parametrize("path,value", [
    (("layers", 0, "type"), "conv"),
    (("layers", 0, "mixer", "rot", "dims"), 8),                 # more than a map's channels
    (("layers", 0, "mixer", "rot", "dims"), 3),
    (("layers", 0, "mixer", "kv_heads"), 3),
    (("layers", 1, "mixer", "vdim"), 6),                        # values that are keys have the keys' size
    (("layers", 2, "mixer", "kv_from"), 2),                     # itself
    (("layers", 2, "mixer", "kv_from"), 1),                     # a layer of the other kind
    (("layers", 2, "mixer", "kv_heads"), 4),                    # another head layout than its source
    (("layers", 2, "mixer", "rot", "base"), 400.0),             # another rotation than its source
    (("layers", 0, "mlp", "router", "top"), 6),
    (("layers", 0, "mlp", "kind"), "dense"),
])
def test_config_reader_refuses(path, value):
    from vllm_omni_draft_amd import config
    cfg = json.loads(json.dumps(CFG))
    node = cfg
    for k in path[:-1]:
        node = node[k]
    node[path[-1]] = value
    with pytest.raises(ValueError):
        config.zopupel_config(cfg)


def test_a_layer_that_reads_another_layers_keys_owns_no_cache():
    from vllm_omni_draft_amd import _lib, config
    from vllm_omni_draft_amd.kv_cache import PAGE, SeqCache
    if not os.path.exists(_lib.lib_path()):
        subprocess.run(["make", "-C", ROOT, "-j8"], check=True)
    mc = config.zopupel_config(CFG)
    c = SeqCache(mc, torch.bfloat16, max_seqs=3, num_pages=7, max_seq_len=4 * PAGE, device="cpu")
    assert c.has_pages and sorted(c.k) == sorted(c.v) == [0, 1] and not c.state and c.kv_source == {2: 0}
    assert c.k[0].shape == (7, 2 * 2, PAGE, 6) and c.v[0].shape == (7, 2, PAGE, 10)     # two key rows per kv head
    assert c.k[1].shape == c.v[1].shape == (7, 1, PAGE, 8)
    assert c.keys_of(2) is c.k[0] and c.values_of(2) is c.v[0] and c.keys_of(1) is c.k[1]
    assert c.nbytes() == 2 * (c.k[0].numel() + c.v[0].numel() + 2 * c.k[1].numel())


def test_weights_are_stacked_per_layer():
    from vllm_omni_draft_amd import config, weights
    st = Z.random_tensors(CFG, 3)
    mc = config.zopupel_config(CFG)
    w = weights.seq_from_state_dict(mc, st, "cpu", torch.float32)
    a, b, c = w.layers
    assert a.w_in.shape == (4 * 2 * 6 + 2 * 2 * 6 + 2 * 10, 40) and torch.equal(a.w_in[-20:], st["l0.mix.v"])
    assert abs(a.diff_lambda - Z.diff_lambda(Z.sub(st, "l0.mix."), 0.25)) < 1e-6 and a.w_in_bias is None and a.sinks is None
    assert a.inv_freq.dtype == torch.float64 and torch.equal(a.inv_freq, Z.frequencies(CFG["layers"][0]["mixer"]["rot"])[0])
    assert a.rot_mag == 1.0 and a.router_bias.dtype == torch.float32 and torch.equal(a.router_bias, st["l0.mlp.router.b"])
    assert a.w_gate_up.shape == (5, 40, 40) and a.w_down_e.shape == (5, 40, 20) and a.w_shared_in.shape == (24, 40)
    assert a.w_shared_gate is None
    assert b.w_in.shape == (3 * 8 + 8, 40) and torch.equal(b.w_in_bias, torch.cat([st["l1.mix.q.b"], st["l1.mix.k.b"]]))
    assert b.q_norm_w.shape == (24,) and b.k_norm_w.shape == (8,) and torch.equal(b.w_o_bias, st["l1.mix.o.b"])
    assert torch.equal(b.sinks, torch.zeros(3)) and b.norm2_w is None and b.rot_mag == 0.1 * math.log(4.0) + 1.0
    assert c.w_in.shape == (4 * 2 * 6, 40) and c.k_norm_w is None and c.w_shared_in is None
    assert w.head.shape == (70, 40) and w.loop_step is None
    st2 = weights.seq_random_state(mc, 0)
    assert {k: tuple(v.shape) for k, v in st2.items()} == {k: tuple(v.shape) for k, v in st.items()}
    del st["l1.mix.o.b"]
    with pytest.raises(KeyError):
        weights.seq_from_state_dict(mc, st, "cpu", torch.float32)
