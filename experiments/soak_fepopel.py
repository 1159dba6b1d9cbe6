"""Random Fepopel models (layer lists, repeated spans, sizes and constants drawn per seed) under
random schedules (portions of prompts beside single tokens, fewer slots than requests) against the
plain CPU model of oracle/fepopel.py, in float32 or (third argument "bf16") bfloat16, where most
rows must stay close.  Prints one line per seed; exits non-zero if any row is off.

    python experiments/soak_fepopel.py [first_seed [n_seeds [bf16]]]
"""
import os
import random
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
from oracle import fepopel as P  # noqa: E402


def draw_model(rng):
    def feed_forward():
        u = rng.random()
        if u < 0.15:
            return None
        if u < 0.4:
            return {"kind": "dense", "ff": rng.choice([8, 20, 32, 72, 96])}
        n = rng.choice([1, 2, 3, 4, 5, 8, 9, 16])
        out = {"kind": "moe", "expert": {"ff": rng.choice([8, 12, 20, 32, 64])},
               "router": {"experts": n, "top": rng.randint(1, min(n, 4)), "scale": rng.choice([0.5, 1.0, 1.5, 2.5])}}
        if rng.random() < 0.75:
            out["shared"] = {"ff": rng.choice([4, 12, 32, 64, 128])}
        return out

    def latent():
        rot_dim = rng.choice([0, 2, 4, 6, 8, 16, 32])
        m = dict(heads=rng.choice([1, 2, 3, 4, 6, 8]), dim=rng.choice([4, 8, 12, 16, 24, 32]), rot_dim=rot_dim,
                 vdim=rng.choice([4, 6, 8, 16, 20, 32, 40]), kv_rank=rng.choice([8, 13, 16, 24, 40, 64, 72]),
                 scale=rng.choice([0.1, 0.2, 0.25, 0.5]), rot={"dims": rot_dim, "base": rng.choice([100.0, 1e4, 1e6])})
        return {"type": "latent_attention", "mixer": m, "mlp": feed_forward()}

    def chunked():
        G = rng.choice([1, 2, 3, 4])
        m = dict(heads=G * rng.choice([1, 2, 4]), kv_heads=G, dim=rng.choice([4, 8, 12, 20, 32, 64]),
                 vdim=rng.choice([4, 8, 12, 24, 32, 72]), scale=rng.choice([0.1, 0.2, 0.3]),
                 softcap=rng.choice([0.5, 5.0, 15.0, 50.0]), mask={"size": rng.choice([1, 3, 8, 16, 40, 70, 100, 400])})
        return {"type": "attention", "mixer": m, "mlp": feed_forward()}

    n = rng.randint(1, 6)
    layers = [rng.choice([latent, latent, chunked])() for _ in range(n)]
    cfg = {"architecture": "Fepopel", "width": rng.choice([24, 40, 56, 64, 72, 96, 128, 160, 256, 320, 516]),
           "vocab": rng.randint(40, 700), "norm": {"eps": rng.choice([1e-5, 1e-6])},
           "embedding": {"scale": rng.choice([1.0, 3.0, 12.0])}, "layers": layers}
    if rng.random() < 0.8:
        a = rng.randint(0, n - 1)
        cfg["loop"] = {"start": a, "stop": rng.randint(a + 1, n), "times": rng.choice([1, 2, 2, 3])}
    return cfg


def rel(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return ((a - b).pow(2).mean().sqrt() / b.pow(2).mean().sqrt().clamp_min(1e-30)).item()


def run(seed, dtype=torch.float32):
    from vllm_omni_draft_amd import config, weights
    from vllm_omni_draft_amd.seq_engine import SeqEngine, SeqEngineConfig
    rng = random.Random(seed)
    cfg = draw_model(rng)
    st = P.random_tensors(cfg, seed)
    mc = config.fepopel_config(cfg, {k: tuple(v.shape) for k, v in st.items()})
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
    kinds = "".join(l["type"][0] for l in cfg["layers"])
    loop = cfg.get("loop")
    span = f" span {loop['start']}-{loop['stop']} x{loop['times']}" if loop else ""
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
