"""The Puguzen decoder family on the GPU against the plain CPU restatement in oracle/puguzen.py:
every mechanism alone through its entry point, then whole models through the engine (prompts
whole, token by token, in portions, in mixed batches, over reused slots and pages) and through
the worker and scheduler.  Small random models of several shapes; where random weights would hide
a fault (one far key among many, a window's edge) the inputs are made so that it shows."""
import pytest
import torch

from oracle import puguzen as P

pytestmark = pytest.mark.gpu

DEV = "cuda"


def dev(t, dtype=None):
    return t.to(dtype or t.dtype).contiguous().to(DEV)


def i32(x):
    return torch.tensor(x, dtype=torch.int32, device=DEV)


def rel(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return ((a - b).pow(2).mean().sqrt() / b.pow(2).mean().sqrt().clamp_min(1e-30)).item()


# ------------------------------------------------------------------ model shapes
def layer(kind, **kw):
    ff = kw.pop("ff", 96)
    m = dict(heads=kw.pop("heads", 2), dim=kw.pop("dim", 16), vdim=kw.pop("vdim", 16))
    if kind == "retention":
        m["decay"] = kw.pop("decay", [1 - 2.0 ** -(3 + i) for i in range(m["heads"])])
        m["rot"] = {"dims": kw.pop("rot_dims", m["dim"]), "base": kw.pop("base", 10000.0)}
    elif kind == "gla":
        m["tau"] = kw.pop("tau", 8.0)
        m["rank"] = kw.pop("rank", 4)
    else:
        m["kv_heads"] = kw.pop("kv_heads", 1)
        m["rot"] = {"dims": kw.pop("rot_dims", m["dim"]), "base": kw.pop("base", 10000.0)}
        m["scale"] = kw.pop("scale", 0.25)
        m["mask"] = {"size": kw.pop("window", 9), "pool": kw.pop("pool", 4)}
    assert not kw, kw
    return {"type": kind, "mixer": m, "mlp": {"kind": "dense", "ff": ff} if ff else None}


def model_cfg(layers, width=64, vocab=96, eps=1e-5):
    return {"architecture": "Puguzen", "width": width, "vocab": vocab, "norm": {"eps": eps}, "layers": layers}


SHAPES = {
    "three_kinds": model_cfg([layer("retention"), layer("attention"), layer("gla")]),
    # sizes that divide nothing: odd head counts, partial rotary, a pool that does not divide a page
    "odd": model_cfg([layer("attention", heads=6, kv_heads=3, dim=24, vdim=40, rot_dims=8, window=7, pool=5, ff=100),
                      layer("gla", heads=3, dim=20, vdim=24, rank=3, tau=3.0, ff=0),
                      layer("retention", heads=3, dim=24, vdim=8, rot_dims=12, ff=52)],
                     width=72, vocab=130, eps=1e-6),
    # values that often coincide, made different; window 1, pool 1, one head
    "ones": model_cfg([layer("attention", heads=1, kv_heads=1, dim=8, vdim=12, window=1, pool=1, ff=0),
                       layer("retention", heads=1, dim=40, vdim=72, rot_dims=2, decay=[0.875], ff=24),
                       layer("attention", heads=4, kv_heads=4, dim=16, vdim=8, window=20, pool=32, ff=24)],
                      width=40, vocab=50),
    # widths that are multiples of 32: bfloat16 serving takes the tiled linear kernels everywhere
    # (with a stacked input matrix of an odd number of rows, and a vocabulary that is no multiple of 4)
    "aligned": model_cfg([layer("gla", heads=4, dim=32, vdim=16, rank=5, ff=160),
                          layer("attention", heads=4, kv_heads=2, dim=32, vdim=24, window=12, pool=2, ff=64),
                          layer("retention", heads=2, dim=16, vdim=48, ff=0)], width=128, vocab=178),
    "wide_heads": model_cfg([layer("gla", heads=2, dim=136, vdim=80, rank=5),
                             layer("attention", heads=2, kv_heads=1, dim=72, vdim=136, window=33, pool=3)],
                            width=48, vocab=64),
}


def build(cfg, dtype=torch.float32, seed=0, tiled=True, **eng_kw):
    from vllm_omni_draft_amd import config, weights
    from vllm_omni_draft_amd.seq_engine import SeqEngine, SeqEngineConfig
    st = P.random_model(cfg, seed)
    mc = config.puguzen_config(cfg, {k: tuple(v.shape) for k, v in st.items()})
    w = weights.seq_from_state_dict(mc, st, DEV, dtype, tiled=tiled)
    kw = dict(max_seqs=4, max_tokens=1024)
    kw.update(eng_kw)
    return st, SeqEngine(w, SeqEngineConfig(**kw))


def prompt(cfg, n, seed=0):
    g = torch.Generator().manual_seed(1000 + seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


def oracle_logits(cfg, st, toks):
    return P.forward(cfg, st, toks, P.Sequence(cfg))


# ------------------------------------------------------------------ mechanisms alone
@pytest.mark.parametrize("M,N,K", [(1, 7, 5), (3, 130, 72), (16, 128, 16), (17, 33, 100), (70, 64, 64)])
@pytest.mark.parametrize("wdt", [torch.float32, torch.bfloat16])
def test_matmul_rows(M, N, K, wdt):
    from vllm_omni_draft_amd import ops
    g = torch.Generator().manual_seed(M * 1000 + N)
    x, x2 = torch.randn(M, K, generator=g), torch.randn(M, K, generator=g)
    w, b = torch.randn(N, K, generator=g).to(wdt), torch.randn(N, generator=g)
    rd = (lambda t: t.to(torch.bfloat16).double()) if wdt == torch.bfloat16 else (lambda t: t.double())
    y = ops.matmul_rows(dev(x), dev(w), dev(b))
    assert rel(y, rd(x) @ w.double().T + b.double()) < 2e-6
    y2 = ops.matmul_rows(dev(x), dev(w), None, dev(x2))
    assert rel(y2, rd(torch.relu(x) * x2) @ w.double().T) < 2e-6
    # a row's bits do not depend on how many rows share the launch
    y1 = ops.matmul_rows(dev(x[:1]), dev(w), dev(b))
    assert torch.equal(y1[0], y[0])


@pytest.mark.parametrize("W", [5, 72, 1000])
def test_rmsnorm_rows(W):
    from vllm_omni_draft_amd import ops
    g = torch.Generator().manual_seed(W)
    x, w = torch.randn(6, W, generator=g) * 3, torch.randn(W, generator=g) * 0.2
    out = ops.rmsnorm_rows(dev(x), dev(w), 1e-5, offset=1.0)
    assert rel(out, P.offset_rms_norm(x.double(), w.double(), 1e-5)) < 1e-6
    rows = i32([4, 0])
    out, out_b = ops.rmsnorm_rows(dev(x), dev(w), 1e-3, offset=0.0, rows=rows, bf16_copy=True)
    assert rel(out, P.unit_rms(x.double()[[4, 0]], 1e-3) * w.double()) < 1e-6
    assert torch.equal(out_b, out.to(torch.bfloat16))


@pytest.mark.parametrize("layout,dk,dims", [(0, 16, 16), (0, 24, 12), (1, 24, 8), (1, 70, 70), (1, 8, 0)])
def test_head_prep_rotary_norm_scale(layout, dk, dims):
    from vllm_omni_draft_amd import ops
    g = torch.Generator().manual_seed(dk)
    n, Hq, Hk = 5, 3, 2
    q, k = torch.randn(n, Hq * dk, generator=g), torch.randn(n, Hk * dk, generator=g)
    pos = torch.tensor([0, 1, 7, 1000, 52341])
    fn = P.rotate_interleaved_layout if layout else P.rotate_half_layout
    base = 5000.0
    inv = dev(torch.tensor(base, dtype=torch.float64) ** (-2.0 * torch.arange(dims // 2, dtype=torch.float64) / max(dims, 1)))
    for unit in (False, True):
        qd, kd = dev(q), dev(k)
        ops.head_prep(qd, kd, i32(pos.tolist()), Hq, Hk, dk, rot_dims=dims, rot_layout=layout,
                      inv_freq=inv if dims else None, unit_norm=unit, eps=1e-4, q_scale=0.5, k_scale=3.0)
        for got, src, H, s in ((qd, q, Hq, 0.5), (kd, k, Hk, 3.0)):
            ref = src.double().view(n, H, dk)
            if dims:
                ref = fn(ref, pos, dims, base)
            if unit:
                ref = P.unit_rms(ref, 1e-4)
            assert rel(got, (ref * s).reshape(n, H * dk)) < 2e-6


def test_sigmoid_power():
    from vllm_omni_draft_amd import ops
    z = torch.linspace(-30, 30, 101).view(1, -1).repeat(2, 1)
    for tau in (1.0, 16.0, 0.5):
        got = ops.sigmoid_power(dev(z), tau)
        assert rel(got, torch.sigmoid(z.double()).pow(1 / tau)) < 2e-6


@pytest.mark.parametrize("H,dk,dv", [(2, 16, 16), (3, 20, 24), (1, 40, 72), (2, 136, 80), (1, 256, 8), (2, 5, 130)])
@pytest.mark.parametrize("per_channel", [False, True])
def test_decay_scan(H, dk, dv, per_channel):
    from vllm_omni_draft_amd import ops
    g = torch.Generator().manual_seed(H * 100 + dk)
    lens = [1, 37, 2, 16]
    n = sum(lens)
    q, k = torch.randn(n, H * dk, generator=g), torch.randn(n, H * dk, generator=g) * dk ** -0.5
    v = torch.randn(n, H * dv, generator=g)
    if per_channel:
        decay = torch.rand(n, H * dk, generator=g) * 0.3 + 0.7
    else:
        decay = torch.rand(H, generator=g) * 0.2 + 0.8
    slots = 5
    state = torch.randn(slots, H, dk, dv, generator=g)      # dirt a fresh sequence must not see
    # entries: slot 3 starts at 0; slot 1 continues (pos 9) from its state; slot 0 fresh; slot 4 continues
    ent = [(3, 0, lens[0], 0), (1, lens[0], lens[1], 9), (0, lens[0] + lens[1], lens[2], 0),
           (4, lens[0] + lens[1] + lens[2], lens[3], 100)]
    sd = dev(state)
    out = ops.decay_scan(dev(q), dev(k), dev(v), dev(decay), sd, i32([list(e) for e in ent]), H, dk, dv)
    for slot, r0, ln, p0 in ent:
        S = state[slot].double().clone() if p0 > 0 else torch.zeros(H, dk, dv, dtype=torch.float64)
        sl = slice(r0, r0 + ln)
        d = (decay[sl].double().view(ln, H, dk) if per_channel
             else decay.double()[None, :, None].expand(ln, H, dk))
        ref = P.decayed_outer_product_scan(q[sl].double().view(ln, H, dk), k[sl].double().view(ln, H, dk),
                                           v[sl].double().view(ln, H, dv), d, S)
        assert rel(out[sl], ref.reshape(ln, H * dv)) < 3e-6
        assert rel(sd[slot], S) < 3e-6
    assert torch.equal(sd[2].cpu(), state[2])               # a slot no entry names is untouched


def test_head_post():
    from vllm_omni_draft_amd import ops
    g = torch.Generator().manual_seed(3)
    n, H, dv = 4, 3, 24
    o, gt, w = torch.randn(n, H * dv, generator=g), torch.randn(n, H * dv, generator=g), torch.randn(dv, generator=g)
    got = ops.head_post(dev(o), dev(gt), H, dv, norm_w=dev(w), unit_norm=True, eps=1e-5, gate="silu")
    ref = (P.unit_rms(o.double().view(n, H, dv), 1e-5) * w.double()).reshape(n, -1) * gt.double() * torch.sigmoid(gt.double())
    assert rel(got, ref) < 2e-6
    got = ops.head_post(dev(o), dev(gt), H, dv, gate="sigmoid")
    assert rel(got, o.double() * torch.sigmoid(gt.double())) < 2e-6


def test_gated_residual():
    from vllm_omni_draft_amd import ops
    g = torch.Generator().manual_seed(4)
    x, z1, z2, a, b = (torch.randn(3, 50, generator=g) for _ in range(5))
    xd = dev(x)
    ops.gated_residual(xd, dev(z1), dev(a), dev(z2), dev(b))
    assert rel(xd, x + torch.sigmoid(z1) * a + torch.sigmoid(z2) * b) < 1e-6
    xd = dev(x)
    ops.gated_residual(xd, dev(z1), dev(a))
    assert rel(xd, x + torch.sigmoid(z1) * a) < 1e-6
    c1, c2 = torch.randn(50, generator=g), torch.randn(50, generator=g)
    xd = dev(x)
    ops.gated_residual(xd, dev(z1), dev(a), dev(z2), dev(b), dev(c1), dev(c2))
    assert rel(xd, x + torch.sigmoid(z1 + c1) * a + torch.sigmoid(z2 + c2) * b) < 1e-6
    # the fused form: the same update, then the next norm
    w = torch.randn(50, generator=g) * 0.1
    xd = dev(x)
    h, h_b = ops.gated_residual_norm(xd, dev(z1), dev(a), dev(w), 1e-5, dev(z2), dev(b), dev(c1), dev(c2))
    xr = x + torch.sigmoid(z1 + c1) * a + torch.sigmoid(z2 + c2) * b
    assert rel(xd, xr) < 1e-6 and rel(h, P.offset_rms_norm(xr.double(), w.double(), 1e-5)) < 1e-6
    assert torch.equal(h_b, h.to(torch.bfloat16))
    act = ops.relu_mul_rows(dev(z1), dev(z2))
    assert torch.equal(act.cpu(), (torch.relu(z1) * z2).to(torch.bfloat16))


class _AttnBed:
    """A window layer's caches over scattered pages, filled through head_prep."""

    def __init__(self, G, dk, dv, pool, n_tokens, dtype=torch.float32, seed=0):
        from vllm_omni_draft_amd import ops
        self.ops, self.G, self.dk, self.dv, self.pool = ops, G, dk, dv, pool
        pages = -(-n_tokens // ops.PAGE)
        g = torch.Generator().manual_seed(seed)
        order = torch.randperm(pages + 3, generator=g)[:pages]       # pages out of order, some unused
        self.tables = i32([order.tolist(), list(range(pages))])      # slot 0 scattered, slot 1 unused here
        ps = ops.pooled_slots_per_page(ops.PAGE, pool)
        n_pg = pages + 3
        self.k = torch.full((n_pg, G, ops.PAGE, dk), 7.0, dtype=dtype, device=DEV)     # dirt everywhere
        self.v = torch.full((n_pg, G, ops.PAGE, dv), -5.0, dtype=dtype, device=DEV)
        self.pk = torch.full((n_pg, G, ps, dk), 9.0, device=DEV)
        self.pv = torch.full((n_pg, G, ps, dv), 9.0, device=DEV)

    def append(self, k, v, pos):
        n = k.shape[0]
        q = torch.zeros(n, self.dk, device=DEV)
        self.ops.head_prep(q, dev(k), i32(pos), 1, self.G, self.dk, v=dev(v), dv=self.dv, k_cache=self.k,
                           v_cache=self.v, row_slot=i32([0] * n), block_tables=self.tables)

    def attend(self, q, pos, H, window, scale, bias):
        n = q.shape[0]
        return self.ops.window_pool_attention(dev(q), self.k, self.v, self.pk, self.pv, i32(pos), i32([0] * n),
                                              self.tables, H, self.G, self.dk, self.dv, window, self.pool, scale,
                                              dev(bias) if bias is not None else None)


@pytest.mark.parametrize("H,G,dk,dv,window,pool", [(2, 1, 16, 16, 9, 4), (6, 3, 24, 40, 7, 5), (1, 1, 8, 12, 1, 1),
                                                   (4, 4, 16, 8, 20, 32), (2, 1, 72, 136, 33, 3), (2, 2, 8, 200, 40, 16),
                                                   (12, 1, 16, 24, 11, 2), (16, 1, 8, 8, 5, 3), (20, 2, 250, 256, 6, 7)])
@pytest.mark.parametrize("step", ["prompt", "decode", "portions"])
def test_window_pool_attention_random(H, G, dk, dv, window, pool, step):
    """Random keys and values over 150 positions: every position against the plain sum, with the
    cache filled in one piece, token by token, or in odd portions."""
    g = torch.Generator().manual_seed(dk + window)
    n = 150
    k, v = torch.randn(n, G * dk, generator=g), torch.randn(n, G * dv, generator=g)
    q, bias = torch.randn(n, H * dk, generator=g), torch.randn(H, generator=g) - 1
    bed = _AttnBed(G, dk, dv, pool, n)
    cuts = {"prompt": [n], "decode": [1] * n, "portions": [2, 13, 1, 31, 2, 64, 5, 2, 30]}[step]
    assert sum(cuts) == n
    out, at = [], 0
    for c in cuts:
        pos = list(range(at, at + c))
        bed.append(k[at:at + c], v[at:at + c], pos)
        out.append(bed.attend(q[at:at + c], pos, H, window, 0.3, bias))
        at += c
    out = torch.cat(out).cpu().double().view(n, H, dv)
    K, V, Q = k.double().view(n, G, dk), v.double().view(n, G, dv), q.double().view(n, H, dk)
    for i in range(n):
        toks, blocks = P.visible_keys(i, window, pool)
        Kt = torch.stack([K[j] for j in toks] + [K[b * pool:(b + 1) * pool].mean(0) for b in blocks])
        Vt = torch.stack([V[j] for j in toks] + [V[b * pool:(b + 1) * pool].mean(0) for b in blocks])
        for h in range(H):
            gi = h // (H // G)
            w = torch.sigmoid(Kt[:, gi] @ Q[i, h] * 0.3 + bias[h].double())
            assert rel(out[i, h], w @ Vt[:, gi]) < 5e-6, (i, h)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_window_pool_attention_many_keys(dtype):
    """More visible keys than one tile of the kernel holds: rows in small batches (their keys are
    cut over several workgroups) and in large ones (one workgroup walks the tiles) agree with the
    plain sum and with each other."""
    g = torch.Generator().manual_seed(5)
    H, G, dk, dv, window, pool, n = 4, 2, 32, 48, 300, 2, 700
    rd = (lambda t: t.to(torch.bfloat16).float()) if dtype == torch.bfloat16 else (lambda t: t)
    k, v = rd(torch.randn(n, G * dk, generator=g)), rd(torch.randn(n, G * dv, generator=g))
    q, bias = torch.randn(n, H * dk, generator=g), torch.randn(H, generator=g) - 3
    bed = _AttnBed(G, dk, dv, pool, n, dtype)
    bed.append(k, v, list(range(n)))
    big = bed.attend(q, list(range(n)), H, window, 0.2, bias).cpu()           # 700 rows: no cut
    rows = [5, 255, 256, 257, 299, 300, 301, 511, 512, 640, 699]
    small = bed.attend(q[rows], rows, H, window, 0.2, bias).cpu()             # 11 rows: keys cut into tiles
    K, V, Q = k.double().view(n, G, dk), v.double().view(n, G, dv), q.double().view(n, H, dk)
    for a, i in enumerate(rows):
        toks, blocks = P.visible_keys(i, window, pool)
        Kt = torch.stack([K[j] for j in toks] + [K[b * pool:(b + 1) * pool].mean(0) for b in blocks])
        Vt = torch.stack([V[j] for j in toks] + [V[b * pool:(b + 1) * pool].mean(0) for b in blocks])
        for h in range(H):
            w = torch.sigmoid(Kt[:, h // 2] @ Q[i, h] * 0.2 + bias[h].double())
            ref = w @ Vt[:, h // 2]
            assert rel(small[a].view(H, dv)[h], ref) < 5e-6 and rel(big[i].view(H, dv)[h], ref) < 5e-6, (i, h)


@pytest.mark.parametrize("window,pool", [(9, 4), (7, 5), (16, 16), (17, 3), (1, 1), (5, 32)])
@pytest.mark.parametrize("decode", [False, True])
def test_window_pool_attention_sees_exactly_its_keys(window, pool, decode):
    """One-hot keys and values: key j points along channel j and the query at position i along
    channel t, with a large scale and a very negative bias, so the only weight that is not ~0 is
    that of token t (or, for the block that holds t, the block's mean, which keeps 1/pool of the
    score and of the value).  Checks every (i, t): near, far, on page borders, just inside and
    just outside the window, blocks just seen and not yet seen, the first tokens."""
    n = 70
    dk = dv = n
    eye = torch.eye(n)
    bed = _AttnBed(1, dk, dv, pool, n)
    if not decode:
        bed.append(eye, eye, list(range(n)))
    big = 30.0 * pool                              # a pooled hit scores big / pool = 30
    for i in range(n):
        if decode:
            bed.append(eye[i:i + 1], eye[i:i + 1], [i])
        ts = list(range(i + 1))                    # every target t for this position, in one launch
        out = bed.attend(eye[ts] * big, [i] * len(ts), 1, window, 1.0, torch.tensor([-15.0])).cpu()
        toks, blocks = P.visible_keys(i, window, pool)
        for t in ts:
            got = out[t, t].item()
            want = 1.0 if t in toks else (1.0 / pool if t // pool in blocks else 0.0)
            assert abs(got - want) < 1e-4, (i, t, got, want)
            if t in toks or want == 0.0:           # nothing else leaks in
                assert abs(out[t].sum().item() - got) < 1e-3, (i, t)


# ------------------------------------------------------------------ whole models
@pytest.mark.parametrize("shape", sorted(SHAPES))
def test_prompt_logits_match_the_plain_model(shape):
    cfg = SHAPES[shape]
    st, eng = build(cfg)
    toks = prompt(cfg, 83)
    want = list(range(83))
    logits, layers = eng.step([("a", toks, want)], layer_out=True)
    lo = []
    ref = P.forward(cfg, st, toks, P.Sequence(cfg), layer_outputs=lo)
    for i, x in enumerate(lo):
        assert rel(layers[i], x) < 1e-5, f"residual after layer {i}"
    assert rel(logits, ref) < 1e-5


@pytest.mark.parametrize("shape", sorted(SHAPES))
@pytest.mark.parametrize("tiled", [False, True])
def test_bfloat16_serving_stays_close(shape, tiled):
    cfg = SHAPES[shape]
    st, eng = build(cfg, torch.bfloat16, tiled=tiled)
    toks = prompt(cfg, 60)
    logits = eng.step([("a", toks, list(range(60)))])
    assert rel(logits, oracle_logits(cfg, st, toks)) < 0.03
    # 300 rows: more than one call of the many-row linear kernels
    toks = prompt(cfg, 300, 4)
    logits = eng.step([("b", toks, list(range(280, 300)))])
    assert rel(logits, oracle_logits(cfg, st, toks)[280:]) < 0.03


@pytest.mark.parametrize("shape", sorted(SHAPES))
@pytest.mark.parametrize("mode", ["float32", "bfloat16-plain", "bfloat16-tiled"])
def test_cut_anywhere_batched_anyhow(shape, mode):
    """The same three prompts: each alone and whole; token by token; in portions down to two
    tokens; all three in mixed batches.  Logits agree to rounding.  With the plain kernels they
    agree to the bit (every sum is taken in an order fixed by the token's own position); the tiled
    linear kernels have one summation order for up to 16 rows and another above."""
    cfg = SHAPES[shape]
    dtype = torch.float32 if mode == "float32" else torch.bfloat16
    st, eng = build(cfg, dtype, tiled=mode.endswith("tiled"))

    def same(a, b):
        return rel(a, b) < 1e-2 if mode.endswith("tiled") else torch.equal(a, b)

    lens = [71, 19, 40]
    toks = [prompt(cfg, n, i) for i, n in enumerate(lens)]
    whole = []
    for i, t in enumerate(toks):
        whole.append(eng.step([(f"w{i}", t, list(range(len(t))))]).cpu())
        eng.finish(f"w{i}")
    if dtype == torch.float32:
        for i, t in enumerate(toks):
            assert rel(whole[i], oracle_logits(cfg, st, t)) < 1e-5
    # token by token
    rows = [eng.step([("d", [t], [0])]).cpu() for t in toks[1]]
    eng.finish("d")
    assert same(torch.cat(rows), whole[1])
    # portions of changing size
    cuts, at, got = [2, 17, 2, 3, 31, 1, 2, 13], 0, []
    for c in cuts:
        c = min(c, lens[0] - at)
        if c <= 0:
            break
        got.append(eng.step([("p", toks[0][at:at + c], list(range(c)))]).cpu())
        at += c
    assert at == lens[0]
    eng.finish("p")
    assert same(torch.cat(got), whole[0])
    # mixed batches: portions of some beside single tokens of others, requests joining and leaving
    at = [0, 0, 0]
    got = [[], [], []]
    plan = [[(0, 5)], [(0, 2), (1, 7)], [(0, 1), (1, 1), (2, 16)], [(1, 1), (0, 30), (2, 2)], [(2, 1), (1, 1)],
            [(0, 33), (1, 9), (2, 21)]]
    for step in plan:
        ents = []
        for i, c in step:
            c = min(c, lens[i] - at[i])
            ents.append((f"m{i}", toks[i][at[i]:at[i] + c], list(range(c))))
        out = eng.step(ents).cpu()
        o = 0
        for (i, _), e in zip(step, ents):
            got[i].append(out[o:o + len(e[1])])
            o += len(e[1])
            at[i] += len(e[1])
    assert at == lens
    for i in range(3):
        assert same(torch.cat(got[i]), whole[i]), i


def test_slots_and_pages_are_used_again():
    """Four slots, a pool of 12 pages: sixteen requests pass through, each checked against its run
    alone in a fresh engine; the pool would not hold three of them without pages coming back."""
    from vllm_omni_draft_amd.kv_cache import OutOfPages, OutOfSlots
    cfg = SHAPES["three_kinds"]
    st, eng = build(cfg, max_seqs=4, max_tokens=192, max_seq_len=96)
    _, fresh = build(cfg, max_seqs=1, max_tokens=96)
    live = []
    for r in range(16):
        n = 40 + 5 * (r % 9)
        t = prompt(cfg, n, r)
        a = eng.step([(f"r{r}", t[:n // 2], [])])
        b = eng.step([(f"r{r}", t[n // 2:], list(range(n - n // 2)))]).cpu()
        ref = fresh.step([("x", t, list(range(n // 2, n)))]).cpu()
        fresh.finish("x")
        assert a.shape[0] == 0 and torch.equal(b, ref), r
        live.append(f"r{r}")
        if len(live) == 2:
            eng.finish(live.pop(0))
    # the limits are enforced, and a refused step leaves the engine usable
    eng.step([("big", prompt(cfg, 60), [])])
    with pytest.raises(OutOfPages):
        eng.step([("big2", prompt(cfg, 90), [])])
    eng.finish("big2")
    for i in range(2):
        eng.step([(f"s{i}", [1], [])])
    with pytest.raises(OutOfSlots):
        eng.step([("s9", [1], [])])


def test_a_step_larger_than_a_pass():
    cfg = SHAPES["odd"]
    st, eng = build(cfg, max_rows=16)
    _, big = build(cfg)
    ta, tb = prompt(cfg, 50, 1), prompt(cfg, 37, 2)
    want_a, want_b = [0, 15, 16, 49], [36, 3]
    got = eng.step([("a", ta, want_a), ("b", tb, want_b)]).cpu()
    assert eng.passes == 6
    ref = big.step([("a", ta, want_a), ("b", tb, want_b)]).cpu()
    assert torch.equal(got, ref)
    assert rel(got[:4], oracle_logits(cfg, st, ta)[want_a]) < 1e-5


def test_far_tokens_through_recurrent_state():
    """A decay of exactly 1 in one head keeps the first token's contribution for ever: the logits
    600 tokens on still depend on token 0, in the engine as in the plain model."""
    cfg = model_cfg([layer("retention", heads=2, decay=[1.0, 0.5], ff=0), layer("gla", tau=64.0, ff=0)])
    st, eng = build(cfg)
    t1 = prompt(cfg, 600, 5)
    t2 = [(t1[0] + 1) % cfg["vocab"]] + t1[1:]
    eng.step([("a", t1[:599], []), ("b", t2[:599], [])])
    l = eng.step([("a", t1[599:], [0]), ("b", t2[599:], [0])]).cpu()
    r1, r2 = oracle_logits(cfg, st, t1)[-1], oracle_logits(cfg, st, t2)[-1]
    assert rel(l[0], r1) < 2e-5 and rel(l[1], r2) < 2e-5
    assert rel(r1, r2) > 1e-3 and rel(l[0] - l[1], r1 - r2) < 0.1


def test_long_decoding():
    cfg = SHAPES["odd"]
    st, eng = build(cfg, torch.float32)
    toks = prompt(cfg, 260, 9)
    eng.step([("a", toks[:20], [])])
    rows = [eng.step([("a", [t], [0])]) for t in toks[20:]]
    assert rel(torch.cat(rows), oracle_logits(cfg, st, toks)[20:]) < 1e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_decode_steps_replayed_as_graphs(dtype):
    """Decoding steps of one shape replay a captured graph from their third occurrence on; between
    the replays other work runs (a prompt joins, a request leaves, the batch changes shape and
    comes back).  Every step's logits equal those of an engine that launches kernel by kernel."""
    cfg = SHAPES["three_kinds"]
    _, a = build(cfg, dtype, use_graph=True)
    _, b = build(cfg, dtype, use_graph=False)
    toks = [prompt(cfg, 40, i) for i in range(3)]

    def both(entries):
        x, y = a.step(entries).cpu(), b.step(entries).cpu()
        assert torch.equal(x, y)

    both([("r0", toks[0][:9], [8]), ("r1", toks[1][:3], [])])
    for t in range(9, 20):
        both([("r0", [toks[0][t]], [0]), ("r1", [toks[1][t - 6]], [0])])
    both([("r2", toks[2][:17], [16]), ("r0", [toks[0][20]], [0])])          # a prompt beside a decoded token
    for t in range(21, 30):
        both([("r0", [toks[0][t]], [0]), ("r1", [toks[1][t - 7]], []), ("r2", [toks[2][t - 4]], [0])])
    a.finish("r1"), b.finish("r1")
    for t in range(30, 40):
        both([("r2", [toks[2][t - 4]], [0]), ("r0", [toks[0][t]], [0])])    # the two-request shape again
    assert a.graph_replays >= 20 and b.graph_replays == 0


def test_greedy_generation_through_worker_and_scheduler():
    from vllm_omni_draft_amd import config, weights
    from vllm_omni_draft_amd.scheduler import SpecDecodeScheduler
    from vllm_omni_draft_amd.seq_engine import SeqWorker, SeqWorkerConfig
    cfg = SHAPES["three_kinds"]
    st = P.random_model(cfg, 3)
    mc = config.puguzen_config(cfg, {k: tuple(v.shape) for k, v in st.items()})
    worker = SeqWorker(SeqWorkerConfig(weights.seq_from_state_dict(mc, st, DEV, torch.float32), max_num_seqs=3,
                                       max_model_len=128))
    worker.init_device()
    worker.load_model()
    sched = SpecDecodeScheduler.for_worker(worker)
    prompts = [prompt(cfg, n, i) for i, n in enumerate((5, 33, 1, 18, 64, 9, 2))]   # more requests than slots
    reqs = sched.generate(prompts, max_tokens=12)
    assert worker.engine.free_slots == 3
    for p, r in zip(prompts, reqs):
        assert len(r.output_token_ids) == 12 and r.finish_reason == "length"
        seq = P.Sequence(cfg)
        logits = P.forward(cfg, st, p, seq)[-1]
        for tok in r.output_token_ids:
            best = int(logits.argmax())
            if tok != best:                      # legitimate only at a near-tie of the plain model
                top = torch.topk(logits, 2).values
                assert (top[0] - top[1]) / logits.std() < 1e-4
                break
            logits = P.forward(cfg, st, [tok], seq)[-1]


def test_sampling_through_the_worker_is_seeded_per_request():
    from vllm_omni_draft_amd import config, weights
    from vllm_omni_draft_amd.seq_engine import SeqWorker, SeqWorkerConfig
    from vllm_omni_draft_amd.spec_decode_worker import ExecuteModelRequest, SamplingParams, SequenceGroupMetadata
    cfg = SHAPES["three_kinds"]
    st = P.random_model(cfg, 3)
    mc = config.puguzen_config(cfg, {k: tuple(v.shape) for k, v in st.items()})
    w = weights.seq_from_state_dict(mc, st, DEV, torch.float32)   # (bit-equal rows in any batch)

    def run(batch_mates):
        worker = SeqWorker(SeqWorkerConfig(w, max_num_seqs=4, max_model_len=64))
        worker.load_model()
        sp = SamplingParams(temperature=30.0, seed=11, top_k=20)   # hot: tied embeddings make the logits peaked
        metas = [SequenceGroupMetadata("a", True, prompt(cfg, 9, 1), sp, num_prompt_tokens=4)]
        metas += [SequenceGroupMetadata(f"m{i}", True, prompt(cfg, 5 + i, 7 + i),
                                        SamplingParams(temperature=0.7)) for i in range(batch_mates)]
        out, toks = worker.execute_model(ExecuteModelRequest(metas)), []
        assert out.sampled_token_ids[0] == []          # a prompt that is not finished emits nothing
        for _ in range(10):
            metas = [SequenceGroupMetadata(m.request_id, False, sampling_params=m.sampling_params) for m in metas]
            out = worker.execute_model(ExecuteModelRequest(metas))
            toks += out.sampled_token_ids[out.req_id_to_index["a"]]
        return toks

    alone, among = run(0), run(3)
    assert len(alone) == 10 and alone == among
    assert len(set(alone)) > 2
