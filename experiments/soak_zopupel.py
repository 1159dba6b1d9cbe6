"""Random Zopupel models (layer lists, sizes, constants and shared keys drawn per seed) under
random schedules (portions of prompts beside single tokens, fewer slots than requests) against the
plain CPU model of oracle/zopupel.py, in float32 or (third argument "bf16") bfloat16, where most
rows must stay close.  Prints one line per seed; exits non-zero if any row is off.

    python experiments/soak_zopupel.py [first_seed [n_seeds [bf16]]]
"""
import os
import random
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
from oracle import zopupel as P  # noqa: E402


def draw_model(rng):
    def feed_forward():
        if rng.random() < 0.15:
            return None
        n = rng.choice([1, 2, 3, 4, 5, 8, 9, 16])
        out = {"kind": "moe", "expert": {"ff": rng.choice([8, 12, 20, 32, 64])},
               "router": {"experts": n, "top": rng.randint(1, min(n, 4))}}
        if rng.random() < 0.75:
            out["shared"] = {"ff": rng.choice([4, 12, 32, 64, 128])}
        return out

    def rot(dim, blended):
        dims = rng.choice([d for d in (0, 2, 4, 6, 8, 16, 32, 64) if d <= dim])
        sc = {"factor": rng.choice([1.0, 2.0, 4.0, 8.0])}
        if blended:
            sc.update(original=rng.choice([16, 64, 512, 4096]), fast=rng.choice([4.0, 32.0]), slow=rng.choice([0.5, 1.0]))
        return {"dims": dims, "base": rng.choice([100.0, 1e4, 1e6]), "scaling": sc}

    def keyval():
        G, dim = rng.choice([1, 2, 3, 4]), rng.choice([4, 8, 12, 20, 32, 64, 72])
        m = dict(heads=G * rng.choice([1, 2, 4, 8]), kv_heads=G, dim=dim, vdim=dim, scale=rng.choice([0.05, 0.1, 0.2]),
                 rot=rot(dim, True))
        return {"type": "attention_2", "mixer": m, "mlp": feed_forward()}

    def diff(layers):
        sources = [i for i, l in enumerate(layers) if l["type"] == "attention" and "kv_from" not in l["mixer"]]
        if sources and rng.random() < 0.5:
            src = rng.choice(sources)
            m = dict(layers[src]["mixer"], kv_from=src)
        else:
            G, dim = rng.choice([1, 2, 3, 4]), rng.choice([4, 8, 12, 16, 24, 32, 64])
            m = dict(heads=G * rng.choice([1, 2, 4, 8]), kv_heads=G, dim=dim, vdim=rng.choice([4, 8, 12, 24, 32, 72, 136]),
                     scale=rng.choice([0.1, 0.2, 0.3]), diff=rng.choice([0.0, 0.2, 0.5, 0.8]), rot=rot(dim, False))
        return {"type": "attention", "mixer": m, "mlp": feed_forward()}

    layers = []
    for _ in range(rng.randint(1, 7)):
        layers.append(keyval() if rng.random() < 0.5 else diff(layers))
    return {"architecture": "Zopupel", "width": rng.choice([24, 40, 56, 64, 72, 96, 128, 160, 256, 320, 516]),
            "vocab": rng.randint(40, 700), "norm": {"eps": rng.choice([1e-5, 1e-6])},
            "residual_mult": rng.choice([0.2, 0.5, 1.0]), "layers": layers}


def rel(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return ((a - b).pow(2).mean().sqrt() / b.pow(2).mean().sqrt().clamp_min(1e-30)).item()


def run(seed, dtype=torch.float32):
    from vllm_omni_draft_amd import config, weights
    from vllm_omni_draft_amd.seq_engine import SeqEngine, SeqEngineConfig
    rng = random.Random(seed)
    cfg = draw_model(rng)
    st = P.random_tensors(cfg, seed)
    mc = config.zopupel_config(cfg, {k: tuple(v.shape) for k, v in st.items()})
    eng = SeqEngine(weights.seq_from_state_dict(mc, st, "cuda", dtype),
                    SeqEngineConfig(max_seqs=2, max_tokens=512, max_seq_len=256, max_rows=rng.choice([16, 64, 2048])))
    g = torch.Generator().manual_seed(seed)
    reqs = []
    for i in range(4):
        toks = torch.randint(0, cfg["vocab"], (rng.randint(3, 140),), generator=g).tolist()
        reqs.append((str(i), toks, P.forward(cfg, st, toks)))
    waiting, live, worst = list(reqs), [], 0.0
    got = {r[0]: [] for r in reqs}
    while waiting or live:
        while waiting and len(live) < 2:
            live.append([waiting.pop(0), 0])
        entries = []
        for item in live:
            (rid, toks, _), at = item
            if rng.random() < 0.15 and len(live) > 1:
                continue                                  # left out of this step
            n = min(len(toks) - at, rng.choice([1, 1, 2, 3, 7, 16, 17, 40]))
            entries.append((rid, toks[at:at + n], list(range(n))))
            item[1] = at + n
        if not entries:
            continue
        out = eng.step(entries)
        at = 0
        for rid, t, _ in entries:
            got[rid].append(out[at:at + len(t)])
            at += len(t)
        for item in list(live):
            if item[1] == len(item[0][1]):
                eng.finish(item[0][0])
                live.remove(item)
    bad, errs = 0, []
    for rid, toks, want in reqs:
        have = torch.cat(got[rid])
        for r in range(len(toks)):
            e = rel(have[r], want[r])
            errs.append(e)
            worst = max(worst, e)
            bad += e > 2e-4      # (float32 sums through several output norms: errors of a few 1e-5 occur)
    kinds = "".join("k" if l["type"] == "attention_2" else ("s" if "kv_from" in l["mixer"] else "d") for l in cfg["layers"])
    span = ""
    if dtype == torch.bfloat16:
        # (a router's near-tie may fall the other way in bfloat16, and the rows behind it feel that)
        errs.sort()
        bad = int(errs[len(errs) // 2] > 3e-2 or errs[int(len(errs) * 0.9)] > 0.15)
        worst = errs[int(len(errs) * 0.9)]
    print(f"seed {seed}: layers {kinds}{span} width {cfg['width']} worst {worst:.2e} rows off {bad}", flush=True)
    return bad


if __name__ == "__main__":
    first = int(sys.argv[1]) if len(sys.argv) > 1 else 0
    count = int(sys.argv[2]) if len(sys.argv) > 2 else 20
    dt = torch.bfloat16 if len(sys.argv) > 3 and sys.argv[3] == "bf16" else torch.float32
    total = sum(run(s, dt) for s in range(first, first + count))
    sys.exit(1 if total else 0)
