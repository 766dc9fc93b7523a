"""Random Naburax models (layer lists, sizes and constants drawn per seed) under random schedules
(portions of prompts beside single tokens, fewer slots than requests) against the plain CPU model
of oracle/naburax.py, in float32.  Prints one line per seed; exits non-zero if any row is off.

    python experiments/soak_naburax.py [first_seed [n_seeds]]
"""
import os
import random
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
from oracle import naburax as N  # noqa: E402


def draw_model(rng):
    def experts():
        if rng.random() < 0.2:
            return None
        n = rng.choice([1, 2, 3, 4, 5, 8, 9])
        return {"kind": "moe", "expert": {"ff": rng.choice([8, 12, 20, 32, 40])},
                "router": {"experts": n, "top": rng.randint(1, min(n, 3))}}

    def latent():
        rot_dim = rng.choice([0, 2, 4, 6, 8, 16])
        m = dict(heads=rng.choice([1, 2, 3, 4, 6]), dim=rng.choice([4, 8, 12, 16, 24]), rot_dim=rot_dim,
                 vdim=rng.choice([4, 6, 8, 16, 20, 40]), q_rank=rng.randint(5, 40), kv_rank=rng.choice([8, 13, 16, 24, 40, 72]),
                 scale=rng.choice([0.1, 0.25, 0.5]), mask={"size": rng.choice([1, 2, 5, 16, 17, 33, 80])},
                 rot={"dims": rng.choice([d for d in range(0, rot_dim + 1, 2)]), "base": rng.choice([100.0, 1e4, 1e6])})
        if rng.random() < 0.7:
            m["rot"]["scaling"] = {"factor": rng.choice([2.0, 8.0, 40.0]), "original": rng.choice([16, 64, 2048]),
                                   "fast": rng.choice([4.0, 32.0]), "slow": rng.choice([0.5, 1.0])}
        return {"type": "latent_attention", "mixer": m, "mlp": experts()}

    def parallel():
        G = rng.choice([1, 2, 3])
        sg = rng.choice([1, 2, 3])
        sh, sp = sg * rng.choice([1, 2]), rng.choice([4, 6, 8, 12, 24])
        inner = sh * sp
        m = dict(left=dict(heads=G * rng.choice([1, 2, 4]), kv_heads=G, dim=rng.choice([4, 8, 12, 20, 32]),
                           vdim=rng.choice([4, 8, 12, 24, 72]), scale=rng.choice([0.1, 0.3]),
                           mask={"size": rng.choice([1, 3, 8, 16, 40, 70]), "keep_first": rng.choice([0, 0, 1, 4, 9])}),
                 right=dict(heads=sh, vdim=sp, state=rng.choice([4, 8, 12, 20, 48]), groups=sg,
                            conv=rng.choice([1, 2, 3, 4, 5]),
                            norm_groups=rng.choice([d for d in (1, 2, 3, 4) if inner % d == 0])),
                 left_scale=rng.choice([0.5, 0.6, 1.0]), right_scale=rng.choice([0.4, 0.5, 1.0]))
        return {"type": "parallel", "mixer": m, "mlp": experts()}

    layers = [rng.choice([latent, parallel])() for _ in range(rng.randint(1, 4))]
    emb = {"scale": rng.choice([1.0, 3.0, 12.0])}
    if rng.random() < 0.8:
        emb["bigram"] = {"buckets": rng.choice([7, 53, 1021]), "mul_prev": rng.choice([1, 31, 127, 1000003]),
                         "mul_cur": rng.choice([1, 17, 999983])}
    return {"architecture": "Naburax", "width": rng.choice([24, 40, 56, 64, 72, 96, 128]),
            "vocab": rng.randint(40, 300), "norm": {"eps": rng.choice([1e-5, 1e-6])}, "embedding": emb,
            "logit_scale": rng.choice([0.5, 1.0, 2.0]), "layers": layers}


def rel(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return ((a - b).pow(2).mean().sqrt() / b.pow(2).mean().sqrt().clamp_min(1e-30)).item()


def run(seed):
    from vllm_omni_draft_amd import config, weights
    from vllm_omni_draft_amd.seq_engine import SeqEngine, SeqEngineConfig
    rng = random.Random(seed)
    cfg = draw_model(rng)
    st = N.random_tensors(cfg, seed)
    mc = config.naburax_config(cfg, {k: tuple(v.shape) for k, v in st.items()})
    eng = SeqEngine(weights.seq_from_state_dict(mc, st, "cuda", torch.float32),
                    SeqEngineConfig(max_seqs=2, max_tokens=512, max_seq_len=256, max_rows=rng.choice([16, 64, 2048])))
    t64 = {k: v.double() for k, v in st.items()}
    g = torch.Generator().manual_seed(seed)
    reqs = []
    for i in range(4):
        toks = torch.randint(0, cfg["vocab"], (rng.randint(3, 140),), generator=g).tolist()
        reqs.append((str(i), toks, N.forward(cfg, t64, toks, N.Sequence(len(cfg["layers"])))))
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
    bad = 0
    for rid, toks, want in reqs:
        have = torch.cat(got[rid])
        for r in range(len(toks)):
            e = rel(have[r], want[r])
            worst = max(worst, e)
            bad += e > 2e-4      # (float32 sums through several output norms: errors of a few 1e-5 occur)
    kinds = "".join(l["type"][0] for l in cfg["layers"])
    print(f"seed {seed}: layers {kinds} width {cfg['width']} worst {worst:.2e} rows off {bad}", flush=True)
    return bad


if __name__ == "__main__":
    first = int(sys.argv[1]) if len(sys.argv) > 1 else 0
    count = int(sys.argv[2]) if len(sys.argv) > 2 else 20
    total = sum(run(s) for s in range(first, first + count))
    sys.exit(1 if total else 0)
