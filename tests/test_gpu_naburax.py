"""The Naburax decoder family on the GPU against the plain CPU restatement in oracle/naburax.py:
every mechanism alone through its entry point, then whole models through the engine (prompts
whole, token by token, in portions, in mixed batches, over reused slots and pages) and through
the worker and scheduler.  Small random models of several shapes; where random weights would hide
a fault (one far key among many, a kept first token, a window's edge) the inputs are made so
that it shows."""
import pytest
import torch

from oracle import naburax as N

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
def latent(heads=2, dim=8, rot_dim=8, vdim=8, q_rank=12, kv_rank=16, window=9, scale=0.3, rot_dims=None,
           base=10000.0, scaling="default", mlp="default"):
    if scaling == "default":
        scaling = {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}
    m = dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, q_rank=q_rank, kv_rank=kv_rank, scale=scale,
             mask={"size": window}, rot={"dims": rot_dim if rot_dims is None else rot_dims, "base": base})
    if scaling:
        m["rot"]["scaling"] = scaling
    return {"type": "latent_attention", "mixer": m, "mlp": experts() if mlp == "default" else mlp}


def parallel(heads=4, kv_heads=2, dim=8, vdim=8, window=7, keep_first=2, scale=0.3, s_heads=2, s_vdim=8, state=8,
             groups=1, taps=4, norm_groups=1, left_scale=0.7, right_scale=0.4, mlp="default"):
    m = dict(left=dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale,
                       mask={"size": window, "keep_first": keep_first}),
             right=dict(heads=s_heads, vdim=s_vdim, state=state, groups=groups, conv=taps, norm_groups=norm_groups),
             left_scale=left_scale, right_scale=right_scale)
    return {"type": "parallel", "mixer": m, "mlp": experts() if mlp == "default" else mlp}


def experts(n=4, top=2, ff=24):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": n, "top": top}}


def model_cfg(layers, width=32, vocab=80, eps=1e-5, scale=3.0, logit_scale=0.7, bigram="default"):
    if bigram == "default":
        bigram = {"buckets": 53, "mul_prev": 31, "mul_cur": 7}
    emb = {"scale": scale}
    if bigram:
        emb["bigram"] = bigram
    return {"architecture": "Naburax", "width": width, "vocab": vocab, "norm": {"eps": eps}, "embedding": emb,
            "logit_scale": logit_scale, "layers": layers}


SHAPES = {
    "two_kinds": model_cfg([latent(), parallel(), latent(window=5)]),
    # sizes that divide nothing; every pair of sizes that may coincide made different; three experts of
    # five; a recurrence first; several groups and norm groups; a window shorter than the kept tokens
    "odd": model_cfg([parallel(heads=6, kv_heads=3, dim=12, vdim=20, window=3, keep_first=5, s_heads=6, s_vdim=10,
                               state=12, groups=3, taps=3, norm_groups=2, mlp=experts(5, 3, 20)),
                      latent(heads=3, dim=12, rot_dim=6, vdim=10, q_rank=9, kv_rank=21, window=11, rot_dims=4,
                             mlp=None),
                      parallel(heads=2, kv_heads=2, dim=20, vdim=4, window=9, keep_first=0, s_heads=1, s_vdim=24,
                               state=20, taps=2, mlp=experts(3, 1, 10))],
                     width=40, vocab=131, eps=1e-6, bigram={"buckets": 17, "mul_prev": 1000003, "mul_cur": 999983}),
    # window 1, one head, one tap, one expert, no rotation scaling, no bigram table, scales of one
    "ones": model_cfg([latent(heads=1, dim=4, rot_dim=2, vdim=6, q_rank=5, kv_rank=8, window=1, scaling=None,
                              mlp=experts(1, 1, 8)),
                       parallel(heads=1, kv_heads=1, dim=8, vdim=12, window=1, keep_first=1, s_heads=1, s_vdim=4,
                                state=4, taps=1, left_scale=1.0, right_scale=1.0, mlp=None),
                       latent(heads=2, dim=4, rot_dim=0, vdim=6, q_rank=5, kv_rank=8, window=40)],
                      width=24, vocab=50, scale=1.0, logit_scale=1.0, bigram=None),
    # widths that are multiples of 32: bfloat16 serving takes the tiled linear kernels
    "aligned": model_cfg([latent(heads=4, dim=16, rot_dim=16, vdim=8, q_rank=32, kv_rank=64, window=20,
                                 mlp=experts(8, 2, 32)),
                          parallel(heads=4, kv_heads=1, dim=16, vdim=16, window=12, keep_first=3, s_heads=4,
                                   s_vdim=16, state=16, groups=2, norm_groups=4, mlp=experts(8, 2, 32))],
                         width=64, vocab=178),
    # heads wider than a lane group, a latent wider than two tiles of value columns, a wide state
    "wide": model_cfg([latent(heads=2, dim=24, rot_dim=8, vdim=40, q_rank=20, kv_rank=136, window=33),
                       parallel(heads=2, kv_heads=1, dim=72, vdim=136, window=33, keep_first=1, s_heads=2, s_vdim=72,
                                state=40, taps=5)], width=48, vocab=64),
}


def build(cfg, dtype=torch.float32, seed=0, tiled=True, **eng_kw):
    from vllm_omni_draft_amd import config, weights
    from vllm_omni_draft_amd.seq_engine import SeqEngine, SeqEngineConfig
    st = N.random_tensors(cfg, seed)
    mc = config.naburax_config(cfg, {k: tuple(v.shape) for k, v in st.items()})
    w = weights.seq_from_state_dict(mc, st, DEV, dtype, tiled=tiled)
    kw = dict(max_seqs=4, max_tokens=1024)
    kw.update(eng_kw)
    return st, SeqEngine(w, SeqEngineConfig(**kw))


def prompt(cfg, n, seed=0):
    g = torch.Generator().manual_seed(1000 + seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


def f64(st):
    return {k: v.double() for k, v in st.items()}


def oracle_logits(cfg, st, toks, layer_out=None):
    return N.forward(cfg, f64(st), toks, N.Sequence(len(cfg["layers"])), layer_out)


# ------------------------------------------------------------------ mechanisms alone
def test_embed_hashed():
    from vllm_omni_draft_amd import ops
    g = torch.Generator().manual_seed(0)
    V, W, buckets = 70, 36, 13
    table, bg = torch.randn(V, W, generator=g), torch.randn(buckets + 1, W, generator=g)
    toks = torch.randint(0, V, (9,), generator=g).tolist()
    cfg = {"embedding": {"scale": 2.5, "bigram": {"buckets": buckets, "mul_prev": 2000003, "mul_cur": 1999993}}}
    seq = N.Sequence(0)
    want = N.embed(cfg, {"embed": table.double(), "bigram": bg.double()}, toks, seq)
    x = ops.embed_hashed(i32(toks), dev(table), 2.5, i32([-1] + toks[:-1]), dev(bg), 2000003, 1999993)
    assert rel(x, want) < 1e-6
    # a sequence that goes on: the first row pairs with the token before
    want2 = N.embed(cfg, {"embed": table.double(), "bigram": bg.double()}, toks[:3], seq)
    x2 = ops.embed_hashed(i32(toks[:3]), dev(table), 2.5, i32([toks[-1]] + toks[:2]), dev(bg), 2000003, 1999993)
    assert rel(x2, want2) < 1e-6
    x3 = ops.embed_hashed(i32(toks), dev(table), 0.5)
    assert rel(x3, table.double()[toks] * 0.5) < 1e-6


@pytest.mark.parametrize("width,parts", [(5, 1), (72, 3), (1000, 2), (64, 64)])
def test_rmsnorm_parts(width, parts):
    from vllm_omni_draft_amd import ops
    g = torch.Generator().manual_seed(width)
    x, w, z = torch.randn(6, width, generator=g) * 3, torch.randn(width, generator=g), torch.randn(6, width, generator=g)
    out = ops.rmsnorm_parts(dev(x), dev(w), 1e-5, parts)
    want = N.rms_norm(x.double().view(6, parts, -1), None, 1e-5).reshape(6, width) * w.double()
    assert rel(out, want) < 1e-6
    out, out_b = ops.rmsnorm_parts(dev(x), dev(w), 1e-3, parts, gate=dev(z), bf16_copy=True)
    y = x.double() * N.silu(z.double())
    assert rel(out, N.rms_norm(y.view(6, parts, -1), None, 1e-3).reshape(6, width) * w.double()) < 1e-6
    assert torch.equal(out_b, out.to(torch.bfloat16))


@pytest.mark.parametrize("dims,n,scaling", [(8, 8, None), (6, 10, {"factor": 8.0, "original": 128, "fast": 16.0, "slow": 2.0}),
                                            (32, 32, {"factor": 40.0, "original": 4096, "fast": 32.0, "slow": 1.0})])
def test_rope_rows_with_blended_frequencies(dims, n, scaling):
    from vllm_omni_draft_amd import config, ops
    g = torch.Generator().manual_seed(dims)
    H, off = 3, 5
    x = torch.randn(7, H * (off + n), generator=g)
    pos = torch.tensor([0, 1, 2, 63, 64, 5000, 100000])
    f, mag = config.rotary_frequencies(dims, 50000.0, scaling)
    f_ref, mag_ref = N.yarn_frequencies(dims, 50000.0, scaling)
    assert abs(mag - mag_ref) < 1e-12 and torch.allclose(f, f_ref, rtol=1e-12, atol=0)
    if scaling:   # the ends of the ramp: fast pairs keep their frequency, slow ones are divided by the factor
        plain = N.yarn_frequencies(dims, 50000.0, None)[0]
        assert f_ref[0] == plain[0] and abs(f_ref[-1] / plain[-1] - 1 / scaling["factor"]) < 1e-9
    xd = dev(x)
    ops.rope_rows(xd, i32(pos.tolist()), H, off + n, off, dims, dev(f), mag)
    v = x.double().view(7, H, off + n)
    want = torch.cat([v[..., :off], N.rotate_pairs(v[..., off:], pos, dims, f_ref, mag_ref)], -1).reshape(7, -1)
    assert (xd.cpu().double() - want).abs().max() < 2e-6


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
    bt[1] = 0
    ops.cache_append(dev(k.float()), dev(v.float()) if v is not None else None, kc, vc, i32(list(range(n))),
                     i32([0] * n), bt, G, dk, v.shape[1] // G if v is not None else 0)
    return kc, vc, bt


@pytest.mark.parametrize("H,G,dk,dv,window,keep", [(4, 2, 16, 16, 6, 2), (3, 1, 12, 20, 50, 0), (2, 2, 72, 136, 1, 3),
                                                   (9, 1, 8, 8, 17, 40), (16, 2, 8, 300, 5, 1)])
@pytest.mark.parametrize("cdt", [torch.float32, torch.bfloat16])
def test_window_softmax_attention_random(H, G, dk, dv, window, keep, cdt):
    from vllm_omni_draft_amd import ops
    g = torch.Generator().manual_seed(H * 100 + dk)
    n = 45
    q = torch.randn(n, H * dk, generator=g)
    k, v = torch.randn(n, G * dk, generator=g).to(cdt), torch.randn(n, G * dv, generator=g).to(cdt)
    pages = [5, 1, 3]                                  # pages out of order
    kc, vc, bt = fill_cache(k, v, pages, G)
    rows = [0, 1, 2, window - 1, window, window + 1, 16, 31, 32, 44]
    rows = sorted({r for r in rows if 0 <= r < n})
    out = ops.window_softmax_attention(dev(q[rows]), kc, vc, i32(rows), i32([0] * len(rows)), bt, H, G, dk, dv,
                                       window, keep, 0.2)
    want = N.masked_softmax_attention(q.double()[rows].view(-1, H, dk), k.double().view(n, G, dk),
                                      v.double().view(n, G, dv), torch.tensor(rows), 0.2, window, keep)
    assert rel(out, want.reshape(len(rows), -1)) < 3e-6


def test_window_softmax_attention_values_inside_key_rows():
    """Latent attention: the value of a token is the first dv channels of its cached key row."""
    from vllm_omni_draft_amd import ops
    g = torch.Generator().manual_seed(3)
    n, H, dk, dv = 40, 5, 24, 16
    q, k = torch.randn(n, H * dk, generator=g), torch.randn(n, dk, generator=g)
    kc, _, bt = fill_cache(k, None, [2, 0, 1], 1)
    rows = list(range(n))
    out = ops.window_softmax_attention(dev(q), kc, None, i32(rows), i32([0] * n), bt, H, 1, dk, dv, 11, 0, 0.3)
    want = N.masked_softmax_attention(q.double().view(n, H, dk), k.double().view(n, 1, dk),
                                      k.double()[:, :dv].reshape(n, 1, dv), torch.tensor(rows), 0.3, 11, 0)
    assert rel(out, want.reshape(n, -1)) < 3e-6


@pytest.mark.parametrize("window,keep", [(1, 0), (1, 2), (5, 0), (5, 3), (16, 1), (17, 16), (33, 4), (300, 2), (3, 7)])
@pytest.mark.parametrize("decode", [False, True])
def test_window_softmax_attention_sees_exactly_its_keys(window, keep, decode):
    """Key j carries a score far above all others only for the query that looks for j, and value
    one-hot(j): the output of query (i, target j) is one-hot(j) if i sees j, else has no weight
    on j.  Every (position, target) pair near a border: the window's edge, the kept tokens' edge,
    page borders, the sequence's first tokens."""
    from vllm_omni_draft_amd import ops
    n, dk = 70, 8
    dv = n
    # key j = a random unit vector; the query that looks for j is 60 times that vector
    gen = torch.Generator().manual_seed(window * 7 + keep)
    code = torch.randn(n, dk, generator=gen)
    code = code / code.norm(dim=1, keepdim=True)
    k, v = code.clone(), torch.eye(n)
    kc, vc, bt = fill_cache(k, v, [4, 0, 2, 3, 1], 1)
    targets = lambda i: sorted({j for j in (0, 1, keep - 1, keep, keep + 1, i - window - 1, i - window, i - window + 1,
                                            i - window + 2, i - 1, i, 15, 16, 17, 31, 32) if 0 <= j <= i})
    pairs = [(i, j) for i in range(n) for j in targets(i)]
    if decode:      # one launch per query row, as single decoded tokens come
        pairs = [p for p in pairs if p[0] in (0, 1, keep, window - 1, window, window + 1, 16, 33, n - 1) and p[0] < n]
        outs = [ops.window_softmax_attention(dev(code[j:j + 1] * 60), kc, vc, i32([i]), i32([0]), bt, 1, 1, dk, dv,
                                             window, keep, 1.0) for i, j in pairs]
        out = torch.cat(outs).cpu()
    else:
        q = torch.stack([code[j] * 60 for _, j in pairs])
        out = ops.window_softmax_attention(dev(q), kc, vc, i32([i for i, _ in pairs]), i32([0] * len(pairs)), bt, 1,
                                           1, dk, dv, window, keep, 1.0).cpu()
    for r, (i, j) in enumerate(pairs):
        sees = N.visible(i, j, window, keep)
        assert abs(out[r].sum().item() - 1) < 1e-4                  # a softmax: the weights sum to one
        assert torch.all(out[r, i + 1:] == 0), (i, j)               # nothing from the future
        if sees:
            assert out[r, j] > 0.5, (i, j, out[r, j].item())
        else:
            assert out[r, j] == 0, (i, j, out[r, j].item())


@pytest.mark.parametrize("cdt", [torch.float32, torch.bfloat16])
def test_window_softmax_attention_many_keys(cdt):
    """More keys than two tiles, a far key that stands out in the first tile, kept tokens ahead."""
    from vllm_omni_draft_amd import ops
    g = torch.Generator().manual_seed(9)
    n, H, G, dk, dv, window, keep = 700, 2, 1, 16, 24, 640, 3
    q = torch.randn(4, H * dk, generator=g)
    k, v = torch.randn(n, dk, generator=g).to(cdt), torch.randn(n, dv, generator=g).to(cdt)
    k[70] = (q[0, :dk] * 3).to(cdt)                    # row 699 of head 0 finds key 70, just inside its window
    pages = torch.randperm(44, generator=g).tolist()
    kc, vc, bt = fill_cache(k, v, pages, G)
    rows = [699, 698, 650, 300]
    out = ops.window_softmax_attention(dev(q), kc, vc, i32(rows), i32([0] * 4), bt, H, G, dk, dv, window, keep, 0.5)
    want = N.masked_softmax_attention(q.double().view(4, H, dk), k.double().view(n, G, dk), v.double().view(n, G, dv),
                                      torch.tensor(rows), 0.5, window, keep)
    assert rel(out, want.reshape(4, -1)) < 3e-6
    assert rel(out[0, :dv], v[70].double()) < 1e-3     # that key takes all the weight
    # few rows have their keys cut over workgroups and merged; many rows, or no scratch, take them in one sweep
    whole = ops.window_softmax_attention(dev(q), kc, vc, i32(rows), i32([0] * 4), bt, H, G, dk, dv, window, keep, 0.5,
                                         split=False)
    assert rel(whole, want.reshape(4, -1)) < 3e-6 and rel(whole, out) < 2e-6
    many = list(range(600, 700))
    q2 = torch.randn(100, H * dk, generator=g)
    out2 = ops.window_softmax_attention(dev(q2), kc, vc, i32(many), i32([0] * 100), bt, H, G, dk, dv, window, keep, 0.5)
    one = ops.window_softmax_attention(dev(q2[37:38]), kc, vc, i32(many[37:38]), i32([0]), bt, H, G, dk, dv, window,
                                       keep, 0.5)
    assert rel(one[0], out2[37]) < 2e-6


@pytest.mark.parametrize("cdt", [torch.float32, torch.bfloat16])
def test_fused_preparation_equals_its_pieces(cdt):
    """The one-launch preparations of both attention kinds give the values of norm, rotation and
    append run one after the other, in the residual buffers and in the cache."""
    from vllm_omni_draft_amd import config, ops
    g = torch.Generator().manual_seed(5)
    n, qr, rk, dr, dims = 21, 20, 24, 10, 6
    pos, slot = i32(list(range(40, 40 + n))), i32([1] * n)
    bt = torch.zeros(2, 4, dtype=torch.int32, device=DEV)
    bt[1] = i32([3, 0, 2, 1])
    ql, kv = torch.randn(n, qr, generator=g), torch.randn(n, rk + dr, generator=g)
    qw, kw = torch.randn(qr, generator=g).to(cdt), torch.randn(rk, generator=g).to(cdt)
    f, mag = config.rotary_frequencies(dims, 1e4, {"factor": 4.0, "original": 32, "fast": 8.0, "slow": 1.0})
    rnd = cdt == torch.bfloat16
    # pieces
    q1 = ops.rmsnorm_parts(dev(ql), dev(qw), 1e-5, round_bf16=rnd)
    kv1 = dev(kv)
    kv1[:, :rk] = ops.rmsnorm_parts(dev(kv[:, :rk]), dev(kw), 1e-5, round_bf16=rnd)
    ops.rope_rows(kv1, pos, 1, 0, rk, dims, dev(f), mag)
    c1 = torch.zeros(4, 1, PAGE, rk + dr, dtype=cdt, device=DEV)
    ops.cache_append(kv1, None, c1, None, pos, slot, bt, 1, rk + dr, 0)
    # one launch
    q2, kv2, c2 = dev(ql), dev(kv), torch.zeros_like(c1)
    ops.latent_prep(q2, dev(qw), kv2, dev(kw), rk, dr, 1e-5, dims, dev(f), mag, c2, pos, slot, bt)
    assert torch.equal(q1, q2) and torch.equal(kv1, kv2) and torch.equal(c1, c2)
    # q and k normed over the whole projection, k and v appended
    H, G, dk, dv = 6, 3, 12, 20
    q, k, v = torch.randn(n, H * dk, generator=g), torch.randn(n, G * dk, generator=g), torch.randn(n, G * dv, generator=g)
    qnw, knw = torch.randn(H * dk, generator=g).to(cdt), torch.randn(G * dk, generator=g).to(cdt)
    qa, ka = ops.rmsnorm_parts(dev(q), dev(qnw), 1e-5), ops.rmsnorm_parts(dev(k), dev(knw), 1e-5)
    kc1, vc1 = torch.zeros(4, G, PAGE, dk, dtype=cdt, device=DEV), torch.zeros(4, G, PAGE, dv, dtype=cdt, device=DEV)
    ops.cache_append(ka, dev(v), kc1, vc1, pos, slot, bt, G, dk, dv)
    qb, kb, kc2, vc2 = dev(q), dev(k), torch.zeros_like(kc1), torch.zeros_like(vc1)
    ops.qk_norm_append(qb, dev(qnw), kb, dev(knw), dev(v), G, dk, dv, 1e-5, kc2, vc2, pos, slot, bt)
    assert torch.equal(qa, qb) and torch.equal(ka, kb) and torch.equal(kc1, kc2) and torch.equal(vc1, vc2)
    assert rel(qb, N.rms_norm(q.double(), qnw.double(), 1e-5)) < 1e-6


@pytest.mark.parametrize("M,B,N_,K", [(1, 3, 7, 5), (5, 2, 130, 24), (40, 6, 16, 136)])
@pytest.mark.parametrize("wdt", [torch.float32, torch.bfloat16])
def test_matmul_rows_batched(M, B, N_, K, wdt):
    from vllm_omni_draft_amd import ops
    g = torch.Generator().manual_seed(M + K)
    x, w = torch.randn(M, B, K, generator=g), torch.randn(B, N_, K, generator=g).to(wdt)
    xr = x.to(torch.bfloat16).double() if wdt == torch.bfloat16 else x.double()
    y = ops.matmul_rows_batched(dev(x), dev(w))
    assert rel(y, torch.einsum("mbk,bnk->mbn", xr, w.double())) < 2e-6


@pytest.mark.parametrize("C,taps", [(5, 4), (300, 3), (64, 1), (7, 7)])
def test_causal_conv_rows_in_portions(C, taps):
    from vllm_omni_draft_amd import ops
    g = torch.Generator().manual_seed(C)
    n = 23
    x, w, b = torch.randn(n, C, generator=g), torch.randn(C, taps, generator=g), torch.randn(C, generator=g)
    want = N.silu(N.short_conv(x.double(), w.double(), b.double(), {}))
    state = torch.full((3, max(taps - 1, 1), C), 7.0, device=DEV)        # stale: a new sequence must not read it
    cuts = [0, 1, 3, 4, 10, 12, n]                                        # portions of 1, 2, 1, 6, 2, 11 tokens
    outs = []
    for lo, hi in zip(cuts, cuts[1:]):
        # the sequence sits in slot 2, behind another entry's rows in slot 0 that must not leak in
        other = torch.randn(2, C, generator=g)
        xx = torch.cat([other, x[lo:hi]])
        rows = hi - lo
        o = ops.causal_conv_rows(dev(xx), dev(w), dev(b), state, i32([0, 1] + list(range(lo, hi))),
                                 i32([0, 0] + [2] * rows), i32([[0, 0, 2, 0], [2, 2, rows, lo]]))
        outs.append(o[2:])
    assert rel(torch.cat(outs), want) < 1e-6


def ssd_reference(x, B, C, dt, a_log, dt_bias, D, S):
    """x [T, H, P], B, C [T, G, N], dt [T, H]; S [H, N, P] changed in place."""
    T, H, P = x.shape
    G = B.shape[1]
    step = N.softplus(dt + dt_bias)
    y = torch.empty_like(x)
    for t in range(T):
        for h in range(H):
            g = h // (H // G)
            S[h] = torch.exp(-torch.exp(a_log[h]) * step[t, h]) * S[h] + step[t, h] * torch.outer(B[t, g], x[t, h])
            y[t, h] = S[h].T @ C[t, g] + D[h] * x[t, h]
    return y


@pytest.mark.parametrize("H,G,N_,P", [(2, 1, 8, 8), (6, 3, 20, 12), (4, 4, 48, 72), (1, 1, 130, 5)])
def test_ssd_steps_and_scan(H, G, N_, P):
    from vllm_omni_draft_amd import ops
    g = torch.Generator().manual_seed(H * 10 + N_)
    T = 37
    x, B, C = torch.randn(T, H * P, generator=g), torch.randn(T, G * N_, generator=g), torch.randn(T, G * N_, generator=g)
    dt = torch.randn(T, H, generator=g) * 2
    dt[3] = 40.0                                       # a large step: softplus is the identity there, no clamp
    a_log, dt_bias, D = torch.randn(H, generator=g), torch.randn(H, generator=g), torch.randn(H, generator=g)
    S = torch.zeros(H, N_, P, dtype=torch.float64)
    want = ssd_reference(x.double().view(T, H, P), B.double().view(T, G, N_), C.double().view(T, G, N_), dt.double(),
                         a_log.double(), dt_bias.double(), D.double(), S)
    step, decay = ops.ssd_steps(dev(dt), dev(dt_bias), dev(a_log))
    assert rel(step, N.softplus(dt.double() + dt_bias.double())) < 1e-6
    state = torch.full((3, H, N_, P), 5.0, device=DEV)  # stale
    outs = []
    cuts = [0, 2, 3, 20, T]
    for lo, hi in zip(cuts, cuts[1:]):
        outs.append(ops.decay_scan_rows(dev(C[lo:hi]), dev(B[lo:hi]), dev(x[lo:hi]), decay[lo:hi].contiguous(),
                                        step[lo:hi].contiguous(), dev(D), state, i32([[1, 0, hi - lo, lo]]), H, G,
                                        N_, P))
    assert rel(torch.cat(outs), want.reshape(T, -1)) < 2e-6
    assert rel(state[1], S) < 2e-6


@pytest.mark.parametrize("E,top,F,W,rows", [(4, 2, 24, 32, 9), (5, 3, 20, 40, 70), (1, 1, 8, 24, 3), (16, 1, 64, 48, 150),
                                            (7, 7, 10, 20, 5),
                                            # widths that are multiples of 32: bfloat16 takes the matrix-core kernels
                                            (8, 2, 96, 64, 100), (3, 1, 32, 32, 33), (6, 3, 160, 1056, 5),
                                            # many rows per expert: the matrix-core kernels take tiles of 128 rows
                                            (4, 2, 64, 160, 301), (2, 1, 32, 64, 700)])
@pytest.mark.parametrize("wdt", [torch.float32, torch.bfloat16])
def test_routed_experts(E, top, F, W, rows, wdt):
    from vllm_omni_draft_amd import ops
    g = torch.Generator().manual_seed(E * 10 + top)
    x = torch.randn(rows, W, generator=g)
    if wdt == torch.bfloat16:
        x = x.to(wdt).float()
    Wt = {"router": (torch.randn(E, W, generator=g) * W ** -0.5).to(wdt)}    # (logits of order one: no tied scores)
    for e in range(E):
        Wt[f"e{e}.gate"], Wt[f"e{e}.up"] = (torch.randn(F, W, generator=g) * W ** -0.5).to(wdt), \
            (torch.randn(F, W, generator=g) * W ** -0.5).to(wdt)
        Wt[f"e{e}.down"] = (torch.randn(W, F, generator=g) * F ** -0.5).to(wdt)
    mlp = {"router": {"experts": E, "top": top}}
    want = N.routed_experts(x.double(), {k: v.double() for k, v in Wt.items()}, mlp)
    logits = ops.matmul_rows(dev(x), dev(Wt["router"]))
    sel_e, sel_w = ops.moe_route(logits, top)
    s = torch.sigmoid(x.double() @ Wt["router"].double().T)
    assert torch.equal(sel_e.cpu().long().sort(1).values, torch.topk(s, top).indices.sort(1).values)
    gu = torch.stack([torch.cat([Wt[f"e{e}.gate"], Wt[f"e{e}.up"]]) for e in range(E)])
    dn = torch.stack([Wt[f"e{e}.down"] for e in range(E)])
    out = ops.moe_experts(dev(x), sel_e, sel_w, dev(gu), dev(dn))
    assert rel(out.sum(1), want) < (2e-6 if wdt == torch.float32 else 1e-2)
    # a row's results do not depend on the rows around it
    one = ops.moe_experts(dev(x[:1]), sel_e[:1].contiguous(), sel_w[:1].contiguous(), dev(gu), dev(dn))
    if wdt == torch.float32:
        assert torch.equal(one[0], out[0])
    else:       # (a few assignments run as matrix-vector products, many as tiles: bfloat16 rounding apart)
        assert rel(one[0], out[0]) < 1e-2


@pytest.mark.parametrize("E,K,top,wdt", [(5, 40, 3, torch.float32), (16, 1000, 2, torch.bfloat16), (130, 64, 7, torch.float32)])
def test_router_product_and_choice_in_one_launch(E, K, top, wdt):
    from vllm_omni_draft_amd import ops
    g = torch.Generator().manual_seed(E)
    x, w = torch.randn(9, K, generator=g), (torch.randn(E, K, generator=g) * K ** -0.5).to(wdt)
    xr = x.to(torch.bfloat16).double() if wdt == torch.bfloat16 else x.double()
    e, sw, logits = ops.moe_route_rows(dev(x), dev(w), top)
    want = xr @ w.double().T
    assert rel(logits, want) < 2e-6
    tk = torch.topk(torch.sigmoid(want), top)
    assert torch.equal(e.cpu().long(), tk.indices) and rel(sw, tk.values) < 1e-6
    e1, sw1, l1 = ops.moe_route_rows(dev(x[4:5]), dev(w), top)          # a row alone: the same bits
    assert torch.equal(l1[0], logits[4]) and torch.equal(e1[0], e[4]) and torch.equal(sw1[0], sw[4])


def test_router_other_scores():
    from vllm_omni_draft_amd import ops
    g = torch.Generator().manual_seed(1)
    z = torch.randn(6, 11, generator=g)
    z[2, 4] = z[2, 9] = 3.0                            # equals: the lower index goes first
    e, w = ops.moe_route(dev(z), 3, "softmax", True)
    p = torch.softmax(z.double(), 1)
    top = torch.topk(p, 3)
    assert rel(w, top.values / top.values.sum(1, keepdim=True)) < 1e-6
    assert e[2].tolist()[:2] == [4, 9]


def test_postnorm_residual():
    from vllm_omni_draft_amd import ops
    g = torch.Generator().manual_seed(2)
    x, a, b, w = (torch.randn(5, 70, generator=g), torch.randn(15, 70, generator=g), torch.randn(5, 70, generator=g),
                  torch.randn(70, generator=g))
    xd = dev(x)
    ops.postnorm_residual(xd, dev(a), dev(w), 1e-5, n_a=3, sa=0.6, b=dev(b), sb=0.5)
    y = 0.6 * a.double().view(5, 3, 70).sum(1) + 0.5 * b.double()
    assert rel(xd, x.double() + N.rms_norm(y, w.double(), 1e-5)) < 1e-6


# ------------------------------------------------------------------ whole models
@pytest.mark.parametrize("shape", list(SHAPES))
def test_prompt_logits_match_the_plain_model(shape):
    cfg = SHAPES[shape]
    st, eng = build(cfg)
    toks = prompt(cfg, 61)
    lo = []
    want = oracle_logits(cfg, st, toks, lo)
    got, trace = eng.step([("a", toks, list(range(len(toks))))], layer_out=True)
    for i, x in enumerate(lo):
        assert rel(trace[i], x) < 3e-6, f"residual after layer {i}"
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
    exact = dtype == torch.float32 or not tiled

    def same(x, y, what):
        if exact:
            assert torch.equal(x, y), what
        else:
            assert rel(x, y) < 1e-2, what
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


def test_a_far_token_through_the_recurrence_and_a_kept_first_token():
    """The recurrence's decay made (almost) one, so that a token 150 positions back still carries
    weight; and a kept first token whose key every later query finds."""
    cfg = model_cfg([parallel(window=4, keep_first=1, mlp=None)], bigram=None)
    st = N.random_tensors(cfg, 5)
    st["l0.mix.right.A_log"] = torch.full_like(st["l0.mix.right.A_log"], -9.0)
    st["l0.mix.left.q.norm"] *= 4
    from vllm_omni_draft_amd import config, weights
    from vllm_omni_draft_amd.seq_engine import SeqEngine, SeqEngineConfig
    mc = config.naburax_config(cfg)
    eng = SeqEngine(weights.seq_from_state_dict(mc, st, DEV, torch.float32), SeqEngineConfig(max_seqs=2, max_tokens=512))
    base, other = prompt(cfg, 160, 6), prompt(cfg, 160, 6)
    other[0] = (base[0] + 1) % cfg["vocab"]           # only the first token differs
    wa, wb = oracle_logits(cfg, st, base), oracle_logits(cfg, st, other)
    assert rel(wa[-1], wb[-1]) > 1e-3                  # ... and the last position still feels it
    ga = eng.step([("a", base[:100], [])])
    ga = torch.cat([eng.step([("a", [t], [0])]) for t in base[100:]])
    gb = eng.step([("b", other, [159])])
    assert rel(ga[-1], wa[-1]) < 3e-6 and rel(gb[0], wb[-1]) < 3e-6


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
    st = N.random_tensors(cfg, 3)
    mc = config.naburax_config(cfg, {k: tuple(v.shape) for k, v in st.items()})
    worker = SeqWorker(SeqWorkerConfig(weights.seq_from_state_dict(mc, st, DEV, torch.float32), max_num_seqs=3,
                                       max_model_len=128))
    worker.init_device()
    worker.load_model()
    sched = SpecDecodeScheduler.for_worker(worker)
    prompts = [prompt(cfg, n, i) for i, n in enumerate((5, 33, 1, 18, 64, 9, 2))]   # more requests than slots
    reqs = sched.generate(prompts, max_tokens=10)
    assert worker.engine.free_slots == 3
    t64 = f64(st)
    for p, r in zip(prompts, reqs):
        assert len(r.output_token_ids) == 10 and r.finish_reason == "length"
        seq = N.Sequence(len(cfg["layers"]))
        logits = N.forward(cfg, t64, p, seq)[-1]
        for tok in r.output_token_ids:
            best = int(logits.argmax())
            if tok != best:                      # legitimate only at a near-tie of the plain model
                top = torch.topk(logits, 2).values
                assert (top[0] - top[1]) / logits.std() < 1e-4
                break
            logits = N.forward(cfg, t64, [tok], seq)[-1]
