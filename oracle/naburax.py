"""The Naburax decoder family restated in plain torch on the CPU, one function per mechanism.
TEST INFRASTRUCTURE ONLY: slow (token by token where a mechanism is a recurrence or a mask),
and sharing no code with the product package.

A model is a dict (`cfg`) in the layout of its config.json plus a dict of tensors under the
checkpoint's names.  Everything is computed in the dtype of the tensors handed in (float64 for a
reference run).  `Sequence` carries what one sequence keeps between calls, so a prompt can be fed
in portions of any size.

Notation.  A layer is   x <- x + N1(mixer(x));  x <- x + N2(ff(x))   with N(y) = y / rms(y) * w
applied to the sublayer's OUTPUT; the sublayers read the residual x itself.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch


# ------------------------------------------------------------------ small pieces
def rms_norm(x: torch.Tensor, w: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if w is None else y * w


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30))))


def yarn_frequencies(dims: int, base: float, scaling: Optional[dict]):
    """(frequencies [dims/2] float64, factor of cos and sin).  Without `scaling`: base^(-2i/dims), 1.
    With it the frequency of pair i is blended between f_i (fast pairs) and f_i / factor (slow
    pairs) along a linear ramp over the pair index."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = base ** (-2.0 * i / dims)
    if not scaling:
        return f, 1.0
    factor, orig = float(scaling["factor"]), float(scaling["original"])

    def pair_of(turns):   # the pair index whose wavelength makes `turns` turns over `orig` positions
        return dims * math.log(orig / (2 * math.pi * turns)) / (2 * math.log(base))

    lo = max(math.floor(pair_of(float(scaling["fast"]))), 0)
    hi = min(math.ceil(pair_of(float(scaling["slow"]))), dims - 1)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0, 1)
    return f / factor * ramp + f * (1 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_pairs(x: torch.Tensor, pos: torch.Tensor, dims: int, freq: torch.Tensor, mag: float) -> torch.Tensor:
    """x [T, heads, n]; channels (2i, 2i+1), i < dims/2, turn by pos * freq[i]; cos and sin carry `mag`."""
    a = pos.to(torch.float64)[:, None] * freq[None, :]
    c, s = (a.cos() * mag).to(x.dtype)[:, None, :], (a.sin() * mag).to(x.dtype)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def visible(i: int, j: int, window: int, keep_first: int = 0) -> bool:
    """Does position i see position j?"""
    return j <= i and (i - j < window or j < keep_first)


def masked_softmax_attention(q, k, v, pos, scale: float, window: int, keep_first: int = 0):
    """q [T, H, dk] for the positions `pos`; k [n, G, dk], v [n, G, dv] for positions 0..n-1.
    Query head h reads key head h // (H/G).  One (query, head) at a time."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=q.dtype)
    for t in range(T):
        i = int(pos[t])
        js = [j for j in range(i + 1) if visible(i, j, window, keep_first)]
        for h in range(H):
            g = h // (H // G)
            s = torch.stack([(q[t, h] * k[j, g]).sum() for j in js]) * scale
            p = torch.softmax(s, 0)
            out[t, h] = (p[:, None] * torch.stack([v[j, g] for j in js])).sum(0)
    return out


# ------------------------------------------------------------------ mixers
def window_gqa(h, pos, W, m, eps, st):
    """Grouped-query softmax attention, no rotation; q and k are normed over the WHOLE projection
    (all heads at once) with a weight of that size; window with kept first tokens."""
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = rms_norm(h @ W["q"].T, W["q.norm"], eps).view(T, H, dk)
    k = rms_norm(h @ W["k"].T, W["k.norm"], eps).view(T, G, dk)
    v = (h @ W["v"].T).view(T, G, dv)
    st["k"] = k if st.get("k") is None else torch.cat([st["k"], k])
    st["v"] = v if st.get("v") is None else torch.cat([st["v"], v])
    o = masked_softmax_attention(q, st["k"], st["v"], pos, m["scale"], m["mask"]["size"],
                                 m["mask"].get("keep_first", 0))
    return o.reshape(T, H * dv) @ W["o"].T


def short_conv(u, w, b, st):
    """Causal convolution per channel: u [T, C], w [C, taps] (last column multiplies the current
    token), zeros before the sequence's start; st["conv"] keeps the last taps-1 inputs."""
    taps = w.shape[1]
    hist = st.get("conv")
    if hist is None:
        hist = torch.zeros(taps - 1, u.shape[1], dtype=u.dtype)
    full = torch.cat([hist, u])
    out = torch.stack([(full[t:t + taps] * w.T).sum(0) for t in range(u.shape[0])]) + b
    st["conv"] = full[full.shape[0] - (taps - 1):]
    return out


def ssd_mixer(h, W, m, eps, st):
    """Selective state space with a scalar decay per head (state-space duality form), token by token:
    S <- exp(-exp(A_log) dt) S + dt * B x^T,  y = S^T C + D x, gated by silu(z), then group-normed."""
    H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner, T = H * P, h.shape[0]
    zxbcdt = h @ W["in"].T
    z, xbc, dt = zxbcdt[:, :inner], zxbcdt[:, inner:2 * inner + 2 * G * N], zxbcdt[:, 2 * inner + 2 * G * N:]
    xbc = silu(short_conv(xbc, W["conv"], W["conv.b"], st))
    x = xbc[:, :inner].view(T, H, P)
    B = xbc[:, inner:inner + G * N].view(T, G, N)
    C = xbc[:, inner + G * N:].view(T, G, N)
    dt = softplus(dt + W["dt_bias"])
    S = st.get("S")
    if S is None:
        S = torch.zeros(H, N, P, dtype=h.dtype)
    y = torch.empty(T, H, P, dtype=h.dtype)
    for t in range(T):
        for hh in range(H):
            g = hh // (H // G)
            S[hh] = torch.exp(-torch.exp(W["A_log"][hh]) * dt[t, hh]) * S[hh] + dt[t, hh] * torch.outer(B[t, g], x[t, hh])
            y[t, hh] = S[hh].T @ C[t, g] + W["D"][hh] * x[t, hh]
    st["S"] = S
    y = y.reshape(T, inner) * silu(z)
    ng = m["norm_groups"]
    y = rms_norm(y.view(T, ng, inner // ng), None, eps).reshape(T, inner) * W["norm"]
    return y @ W["o"].T


def parallel_mixer(h, pos, W, m, eps, st):
    left = window_gqa(h, pos, {k[5:]: v for k, v in W.items() if k.startswith("left.")}, m["left"], eps,
                      st.setdefault("left", {}))
    right = ssd_mixer(h, {k[6:]: v for k, v in W.items() if k.startswith("right.")}, m["right"], eps,
                      st.setdefault("right", {}))
    return m["left_scale"] * left + m["right_scale"] * right


def latent_attention(h, pos, W, m, eps, st):
    """Keys and values of all heads are expanded from one small latent per token; one rotated key
    part is shared by the heads.  Written in the expanded (non-absorbed) form."""
    H, dn, dr, dv, rk = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    T = h.shape[0]
    rot = m["rot"]
    freq, mag = yarn_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
    q = (rms_norm(h @ W["dq"].T, W["dq.norm"], eps) @ W["uq"].T).view(T, H, dn + dr)
    q = torch.cat([q[..., :dn], rotate_pairs(q[..., dn:], pos, rot["dims"], freq, mag)], -1)
    kv = h @ W["dkv"].T
    c = rms_norm(kv[:, :rk], W["dkv.norm"], eps)
    kr = rotate_pairs(kv[:, None, rk:], pos, rot["dims"], freq, mag)          # [T, 1, dr]
    st["c"] = c if st.get("c") is None else torch.cat([st["c"], c])
    st["kr"] = kr if st.get("kr") is None else torch.cat([st["kr"], kr])
    n = st["c"].shape[0]
    k = torch.cat([(st["c"] @ W["uk"].T).view(n, H, dn), st["kr"].expand(n, H, dr)], -1)
    v = (st["c"] @ W["uv"].T).view(n, H, dv)
    o = masked_softmax_attention(q, k, v, pos, m["scale"], m["mask"]["size"], 0)
    return o.reshape(T, H * dv) @ W["o"].T


# ------------------------------------------------------------------ feed-forward
def routed_experts(h, W, mlp):
    """Sigmoid router; the `top` largest scores choose the experts; a score scales its expert's
    INPUT; nothing is renormalised."""
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    s = torch.sigmoid(h @ W["router"].T)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e in torch.topk(s[t], top).indices.tolist():
            u = s[t, e] * h[t]
            out[t] += W[f"e{e}.down"] @ (silu(W[f"e{e}.gate"] @ u) * (W[f"e{e}.up"] @ u))
    return out


# ------------------------------------------------------------------ the model
class Sequence:
    def __init__(self, n_layers: int):
        self.n = 0
        self.prev: Optional[int] = None
        self.layers: List[dict] = [{} for _ in range(n_layers)]


def embed(cfg, tensors, tokens: List[int], seq: Sequence):
    e = cfg["embedding"]
    x = tensors["embed"][tokens] * e["scale"]
    bg = e.get("bigram")
    if bg:
        rows, prev = [], seq.prev
        for t in tokens:
            rows.append(bg["buckets"] if prev is None else (prev * bg["mul_prev"] + t * bg["mul_cur"]) % bg["buckets"])
            prev = t
        x = x + tensors["bigram"][rows]
    seq.prev = tokens[-1]
    return x


def forward(cfg, tensors: Dict[str, torch.Tensor], tokens: List[int], seq: Sequence, layer_out=None):
    """Feeds `tokens` (the sequence's next ones) and returns the logits of every fed token."""
    eps = cfg["norm"]["eps"]
    x = embed(cfg, tensors, tokens, seq)
    pos = torch.arange(seq.n, seq.n + len(tokens))
    for i, l in enumerate(cfg["layers"]):
        W = {k[len(f"l{i}.mix."):]: v for k, v in tensors.items() if k.startswith(f"l{i}.mix.")}
        if l["type"] == "parallel":
            a = parallel_mixer(x, pos, W, l["mixer"], eps, seq.layers[i])
        elif l["type"] == "latent_attention":
            a = latent_attention(x, pos, W, l["mixer"], eps, seq.layers[i])
        else:
            raise ValueError(l["type"])
        x = x + rms_norm(a, tensors[f"l{i}.norm1"], eps)
        if l.get("mlp"):
            M = {k[len(f"l{i}.mlp."):]: v for k, v in tensors.items() if k.startswith(f"l{i}.mlp.")}
            x = x + rms_norm(routed_experts(x, M, l["mlp"]), tensors[f"l{i}.norm2"], eps)
        if layer_out is not None:
            layer_out.append(x.clone())
    seq.n += len(tokens)
    return (rms_norm(x, tensors["final.norm"], eps) @ tensors["head"].T) * cfg["logit_scale"]


# ------------------------------------------------------------------ random models for tests
def random_tensors(cfg, seed: int = 0) -> Dict[str, torch.Tensor]:
    """Seeded tensors under the checkpoint's names, as bfloat16 values held in float32."""
    g = torch.Generator().manual_seed(seed)
    Wd, V = cfg["width"], cfg["vocab"]

    def rn(*shape, s=1.0, mean=0.0):
        return ((torch.randn(*shape, generator=g) * s + mean).to(torch.bfloat16)).float()

    t = {"embed": rn(V, Wd, s=0.1), "head": rn(V, Wd, s=Wd ** -0.5), "final.norm": rn(Wd, s=0.1, mean=1.0)}
    bg = cfg["embedding"].get("bigram")
    if bg:
        t["bigram"] = rn(bg["buckets"] + 1, Wd, s=0.5)
    for i, l in enumerate(cfg["layers"]):
        p, m = f"l{i}.", l["mixer"]
        t[p + "norm1"] = rn(Wd, s=0.1, mean=1.0)
        if l["type"] == "latent_attention":
            H, dn, dr, dv, rk = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            qr = m["q_rank"]
            t[p + "mix.dq"], t[p + "mix.dq.norm"] = rn(qr, Wd, s=Wd ** -0.5), rn(qr, s=0.1, mean=1.0)
            t[p + "mix.uq"] = rn(H * (dn + dr), qr, s=2 * qr ** -0.5)
            t[p + "mix.dkv"], t[p + "mix.dkv.norm"] = rn(rk + dr, Wd, s=Wd ** -0.5), rn(rk, s=0.1, mean=1.0)
            t[p + "mix.uk"], t[p + "mix.uv"] = rn(H * dn, rk, s=2 * rk ** -0.5), rn(H * dv, rk, s=rk ** -0.5)
            t[p + "mix.o"] = rn(Wd, H * dv, s=(H * dv) ** -0.5)
        else:
            a, b = m["left"], m["right"]
            H, G, dk, dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            t[p + "mix.left.q"], t[p + "mix.left.k"] = rn(H * dk, Wd, s=Wd ** -0.5), rn(G * dk, Wd, s=Wd ** -0.5)
            t[p + "mix.left.v"] = rn(G * dv, Wd, s=Wd ** -0.5)
            t[p + "mix.left.q.norm"], t[p + "mix.left.k.norm"] = rn(H * dk, s=0.3, mean=2.0), rn(G * dk, s=0.3, mean=2.0)
            t[p + "mix.left.o"] = rn(Wd, H * dv, s=(H * dv) ** -0.5)
            Hs, P, N, Gs, taps = b["heads"], b["vdim"], b["state"], b["groups"], b["conv"]
            inner, ch = Hs * P, Hs * P + 2 * Gs * N
            t[p + "mix.right.in"] = rn(2 * inner + 2 * Gs * N + Hs, Wd, s=Wd ** -0.5)
            t[p + "mix.right.conv"], t[p + "mix.right.conv.b"] = rn(ch, taps, s=0.5), rn(ch, s=0.2)
            t[p + "mix.right.dt_bias"] = rn(Hs, s=0.5, mean=-1.0)
            t[p + "mix.right.A_log"] = rn(Hs, s=0.5, mean=-1.0)
            t[p + "mix.right.D"] = rn(Hs, s=0.5, mean=1.0)
            t[p + "mix.right.norm"] = rn(inner, s=0.1, mean=1.0)
            t[p + "mix.right.o"] = rn(Wd, inner, s=inner ** -0.5)
        mlp = l.get("mlp")
        if mlp:
            F, E = mlp["expert"]["ff"], mlp["router"]["experts"]
            t[p + "norm2"] = rn(Wd, s=0.1, mean=1.0)
            t[p + "mlp.router"] = rn(E, Wd, s=Wd ** -0.5)   # (logits of order one: no saturated, tied scores)
            for e in range(E):
                t[p + f"mlp.e{e}.gate"], t[p + f"mlp.e{e}.up"] = rn(F, Wd, s=Wd ** -0.5), rn(F, Wd, s=Wd ** -0.5)
                t[p + f"mlp.e{e}.down"] = rn(Wd, F, s=F ** -0.5)
    return t
