"""Host-side parts of the Naburax family that need no GPU: the configuration reader and model
registry, the rotary frequency blending against the plain model's, the caches' shapes, and the
plain CPU model's own consistency (a prompt fed whole, in portions or token by token gives the
same logits; the visibility rule; routing)."""
import json
import os
import subprocess

import pytest
import torch

from oracle import naburax as N

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

MOE = {"kind": "moe", "expert": {"ff": 20}, "router": {"experts": 5, "top": 2}}
CFG = {"architecture": "Naburax", "width": 40, "vocab": 70, "norm": {"eps": 1e-6}, "logit_scale": 0.25,
       "embedding": {"scale": 5.0, "bigram": {"buckets": 29, "mul_prev": 11, "mul_cur": 3}},
       "layers": [
           {"type": "latent_attention", "mlp": MOE,
            "mixer": {"heads": 3, "dim": 8, "rot_dim": 4, "vdim": 12, "q_rank": 10, "kv_rank": 14, "scale": 0.4,
                      "mask": {"size": 6},
                      "rot": {"dims": 4, "base": 500.0,
                              "scaling": {"factor": 4.0, "original": 32, "fast": 4.0, "slow": 1.0}}}},
           {"type": "parallel", "mlp": None,
            "mixer": {"left": {"heads": 4, "kv_heads": 2, "dim": 8, "vdim": 6, "scale": 0.5,
                               "mask": {"size": 5, "keep_first": 3}},
                      "right": {"heads": 2, "vdim": 10, "state": 6, "groups": 2, "conv": 3, "norm_groups": 2},
                      "left_scale": 0.75, "right_scale": 0.5}},
       ]}


def test_visibility_rule():
    for window in (1, 2, 5):
        for keep in (0, 1, 3, 9):
            for i in range(20):
                seen = [j for j in range(25) if N.visible(i, j, window, keep)]
                want = sorted(set(range(max(0, i - window + 1), i + 1)) | set(range(min(keep, i + 1))))
                assert seen == want


def test_plain_model_does_not_care_how_a_prompt_is_cut():
    st = {k: v.double() for k, v in N.random_tensors(CFG, 1).items()}
    g = torch.Generator().manual_seed(0)
    toks = torch.randint(0, CFG["vocab"], (40,), generator=g).tolist()
    whole = N.forward(CFG, st, toks, N.Sequence(2))
    for cuts in ([1] * 40, [2, 7, 1, 20, 10], [39, 1]):
        seq, got, at = N.Sequence(2), [], 0
        for c in cuts:
            got.append(N.forward(CFG, st, toks[at:at + c], seq))
            at += c
        assert torch.allclose(torch.cat(got), whole, atol=1e-10, rtol=0)


def test_latent_attention_equals_its_absorbed_form():
    """Scores and values can be taken against the cached latent itself: q' = U_k^T q per head,
    and the weighted latent expanded afterwards.  The plain model uses the expanded form."""
    m = CFG["layers"][0]["mixer"]
    st = {k[len("l0.mix."):]: v.double() for k, v in N.random_tensors(CFG, 2).items() if k.startswith("l0.mix.")}
    g = torch.Generator().manual_seed(1)
    T, H, dn, dr, dv, rk = 17, m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    h = torch.randn(T, CFG["width"], generator=g, dtype=torch.float64)
    pos = torch.arange(T)
    want = N.latent_attention(h, pos, st, m, 1e-6, {})
    freq, mag = N.yarn_frequencies(m["rot"]["dims"], m["rot"]["base"], m["rot"]["scaling"])
    q = (N.rms_norm(h @ st["dq"].T, st["dq.norm"], 1e-6) @ st["uq"].T).view(T, H, dn + dr)
    kv = h @ st["dkv"].T
    c = N.rms_norm(kv[:, :rk], st["dkv.norm"], 1e-6)
    kr = N.rotate_pairs(kv[:, None, rk:], pos, m["rot"]["dims"], freq, mag)
    qa = torch.einsum("thd,hdr->thr", q[..., :dn], st["uk"].view(H, dn, rk))
    qe = torch.cat([qa, N.rotate_pairs(q[..., dn:], pos, m["rot"]["dims"], freq, mag)], -1)
    rows = torch.cat([c, kr[:, 0]], -1)[:, None, :]
    oc = N.masked_softmax_attention(qe, rows, c[:, None, :], pos, m["scale"], m["mask"]["size"], 0)
    o = torch.einsum("thr,hvr->thv", oc, st["uv"].view(H, dv, rk)).reshape(T, H * dv)
    assert torch.allclose(o @ st["o"].T, want, atol=1e-10, rtol=0)


def test_rotary_frequency_blending():
    from vllm_omni_draft_amd import config
    for dims, base, sc in [(4, 500.0, CFG["layers"][0]["mixer"]["rot"]["scaling"]), (64, 1e6, None),
                           (64, 1e4, {"factor": 32.0, "original": 4096, "fast": 32.0, "slow": 1.0}),
                           (16, 1e4, {"factor": 2.0, "original": 8, "fast": 100.0, "slow": 0.001})]:
        f, mag = config.rotary_frequencies(dims, base, sc)
        fr, magr = N.yarn_frequencies(dims, base, sc)
        assert torch.allclose(f, fr, rtol=1e-13, atol=0) and abs(mag - magr) < 1e-13
        assert f.dtype == torch.float64 and bool((f[1:] <= f[:-1]).all())


def test_config_reader_and_registry(tmp_path):
    from safetensors.torch import save_file
    from vllm_omni_draft_amd import config
    st = N.random_tensors(CFG, 2)
    cfg = json.loads(json.dumps(CFG))
    cfg["layers"][0]["mixer"]["q_rank"] = 99          # the tensor's shape wins
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in st.items()}, str(tmp_path / "model.safetensors"))
    mc = config.load_model_config(str(tmp_path))
    assert isinstance(mc, config.SeqModelConfig) and (mc.arch, mc.block, mc.n_layers) == ("naburax", "postnorm", 2)
    assert (mc.embed_scale, mc.logit_scale, mc.tied_head, mc.norm_eps) == (5.0, 0.25, False, 1e-6)
    assert mc.bigram == {"buckets": 29, "mul_prev": 11, "mul_cur": 3}
    a, b = (l.mixer for l in mc.layers)
    assert (a.kind, a.heads, a.dim, a.rot_dim, a.vdim, a.q_rank, a.kv_rank, a.window, a.rot_dims, a.rot_base) == \
        ("latent_attention", 3, 8, 4, 12, 10, 14, 6, 4, 500.0)
    assert a.rot_scaling["factor"] == 4.0 and a.rot_layout == "interleaved"
    assert (b.kind, b.heads, b.kv_heads, b.dim, b.vdim, b.window, b.keep_first, b.left_scale, b.right_scale) == \
        ("parallel", 4, 2, 8, 6, 5, 3, 0.75, 0.5)
    s = b.ssd
    assert (s.heads, s.vdim, s.state, s.groups, s.taps, s.norm_groups, s.inner, s.conv_channels) == \
        (2, 10, 6, 2, 3, 2, 20, 44)
    e = mc.layers[0].experts
    assert (e.experts, e.top, e.ff, e.score, e.renorm, e.scale_input) == (5, 2, 20, "sigmoid", False, True)
    assert mc.layers[1].experts is None
    assert mc.state_bytes_per_seq() == 4 * (2 * 6 * 10 + 2 * 44)
    assert mc.param_count() == sum(v.numel() for v in st.values())


@pytest.mark.parametrize("path,value", [
    (("layers", 0, "type"), "conv"),
    (("layers", 0, "mixer", "rot", "dims"), 6),                 # more than the rotated channels
    (("layers", 0, "mixer", "rot", "dims"), 3),
    (("layers", 0, "mixer", "mask", "size"), 0),
    (("layers", 0, "mlp", "router", "top"), 6),
    (("layers", 0, "mlp", "kind"), "dense"),
    (("layers", 1, "mixer", "left", "kv_heads"), 3),
    (("layers", 1, "mixer", "right", "groups"), 3),
    (("layers", 1, "mixer", "right", "norm_groups"), 3),
    (("layers", 1, "mixer", "left", "mask", "keep_first"), -1),
])
def test_config_reader_refuses(path, value):
    from vllm_omni_draft_amd import config
    cfg = json.loads(json.dumps(CFG))
    node = cfg
    for k in path[:-1]:
        node = node[k]
    node[path[-1]] = value
    with pytest.raises(ValueError):
        config.naburax_config(cfg)


def test_caches_of_the_two_layer_kinds():
    from vllm_omni_draft_amd import _lib, config
    from vllm_omni_draft_amd.kv_cache import PAGE, SeqCache
    if not os.path.exists(_lib.lib_path()):
        subprocess.run(["make", "-C", ROOT, "-j8"], check=True)
    mc = config.naburax_config(CFG)
    c = SeqCache(mc, torch.bfloat16, max_seqs=3, num_pages=7, max_seq_len=4 * PAGE, device="cpu")
    assert c.has_pages
    assert c.k[0].shape == (7, 1, PAGE, 14 + 4) and 0 not in c.v         # one latent row per token, no values
    assert c.k[1].shape == (7, 2, PAGE, 8) and c.v[1].shape == (7, 2, PAGE, 6)
    assert c.state[1].shape == (3, 2, 6, 10) and c.state[1].dtype == torch.float32
    assert c.conv[1].shape == (3, 2, 44) and c.conv[1].dtype == torch.float32
    assert c.k[0].dtype == torch.bfloat16


def test_routing_takes_the_largest_scores_and_scales_the_input():
    g = torch.Generator().manual_seed(4)
    W = {"router": torch.randn(5, 8, generator=g, dtype=torch.float64)}
    for e in range(5):
        W[f"e{e}.gate"], W[f"e{e}.up"] = (torch.randn(6, 8, generator=g, dtype=torch.float64) for _ in range(2))
        W[f"e{e}.down"] = torch.randn(8, 6, generator=g, dtype=torch.float64)
    h = torch.randn(3, 8, generator=g, dtype=torch.float64)
    out = N.routed_experts(h, W, {"router": {"experts": 5, "top": 2}})
    s = torch.sigmoid(h @ W["router"].T)
    for t in range(3):
        want = 0
        for e in sorted(range(5), key=lambda e: -s[t, e])[:2]:
            u = s[t, e] * h[t]
            want = want + W[f"e{e}.down"] @ (N.silu(W[f"e{e}.gate"] @ u) * (W[f"e{e}.up"] @ u))
        assert torch.allclose(out[t], want, atol=1e-12)
    # the weight is not an output scale: the activation is not linear
    t, e = 0, int(s[0].argmax())
    inside = W[f"e{e}.down"] @ (N.silu(W[f"e{e}.gate"] @ (s[t, e] * h[t])) * (W[f"e{e}.up"] @ (s[t, e] * h[t])))
    outside = s[t, e] * (W[f"e{e}.down"] @ (N.silu(W[f"e{e}.gate"] @ h[t]) * (W[f"e{e}.up"] @ h[t])))
    assert not torch.allclose(inside, outside, atol=1e-6)
