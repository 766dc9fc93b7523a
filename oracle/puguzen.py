"""The Puguzen decoder family restated in plain torch on the CPU, one function per mechanism.
TEST INFRASTRUCTURE ONLY: slow, token by token where the mechanism is a recurrence, and sharing
no code with the product package.

A model is a dict (`cfg`) in the layout of its config.json plus a dict of tensors under the
checkpoint's names.  Every function works in the dtype of its inputs (float64 for a reference
run).  Sequences are handled one at a time; `Sequence` carries what a sequence keeps between
calls (recurrent states and the keys / values of the attention layers), so a prompt can be fed in
portions.

Notation: a layer computes, with h = norm(x),
    x <- x + sigmoid(R1 h + r1) * mixer(h) + sigmoid(R2 h + r2) * ff(h).
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch


# ------------------------------------------------------------------ small pieces
def offset_rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) * (1 + w): the weight is stored around zero."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * (1 + w)


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def _angles(pos: torch.Tensor, dims: int, base: float, dtype) -> torch.Tensor:
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = base ** (-2.0 * i / dims)
    return (pos.to(torch.float64)[:, None] * f[None, :]).to(dtype)          # [T, dims/2]


def rotate_half_layout(x: torch.Tensor, pos: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """x [T, heads, dim]; channel i pairs with channel i + dims/2; channels >= dims untouched."""
    a = _angles(pos, dims, base, x.dtype)[:, None, :]
    u, v = x[..., : dims // 2], x[..., dims // 2: dims]
    out = x.clone()
    out[..., : dims // 2] = u * a.cos() - v * a.sin()
    out[..., dims // 2: dims] = v * a.cos() + u * a.sin()
    return out


def rotate_interleaved_layout(x: torch.Tensor, pos: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """x [T, heads, dim]; channel 2i pairs with channel 2i+1; channels >= dims untouched."""
    a = _angles(pos, dims, base, x.dtype)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * a.cos() - v * a.sin()
    out[..., 1:dims:2] = v * a.cos() + u * a.sin()
    return out


def decayed_outer_product_scan(q, k, v, decay, state):
    """The linear-attention recurrence shared by the two recurrent mixers, one token at a time.
    q, k [T, H, dk], v [T, H, dv], decay [T, H, dk] (a factor per key channel), state [H, dk, dv]
    (changed in place).  S <- diag(decay_t) S + k_t v_t^T;  o_t = S^T q_t."""
    T = q.shape[0]
    out = torch.empty(T, q.shape[1], v.shape[2], dtype=q.dtype)
    for t in range(T):
        state.mul_(decay[t][:, :, None]).add_(k[t][:, :, None] * v[t][:, None, :])
        out[t] = torch.einsum("hkv,hk->hv", state, q[t])
    return out


# ------------------------------------------------------------------ mixers
def retention_mixer(h, pos, W: Dict[str, torch.Tensor], m: dict, eps: float, state):
    """Fixed decay per head, rotate-half rotary on q and k, k scaled after rotation, no softmax."""
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = (h @ W["q"].T).view(T, H, dk)
    k = (h @ W["k"].T).view(T, H, dk)
    v = (h @ W["v"].T).view(T, H, dv)
    q = rotate_half_layout(q, pos, m["rot"]["dims"], m["rot"]["base"])
    k = rotate_half_layout(k, pos, m["rot"]["dims"], m["rot"]["base"]) * dk ** -0.5
    decay = torch.tensor(m["decay"], dtype=h.dtype)[None, :, None].expand(T, H, dk)
    o = decayed_outer_product_scan(q, k, v, decay, state)
    o = unit_rms(o, eps).reshape(T, H * dv)
    g = h @ W["g"].T
    return (o * g * torch.sigmoid(g)) @ W["o"].T


def gla_mixer(h, pos, W: Dict[str, torch.Tensor], m: dict, eps: float, state):
    """A decay per key channel computed from the input through a low-rank pair of matrices."""
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = (h @ W["q"].T).view(T, H, dk) * dk ** -0.5
    k = (h @ W["k"].T).view(T, H, dk)
    v = (h @ W["v"].T).view(T, H, dv)
    z = (h @ W["a1"].T) @ W["a2"].T + W["a2.b"]
    decay = torch.sigmoid(z).pow(1.0 / m["tau"]).view(T, H, dk)
    o = decayed_outer_product_scan(q, k, v, decay, state)
    o = (unit_rms(o, eps) * W["norm"]).reshape(T, H * dv)
    g = h @ W["g"].T
    return (o * g * torch.sigmoid(g)) @ W["o"].T


def visible_keys(i: int, size: int, pool: int):
    """What position i of a windowed layer with pooled blocks sees: the token positions
    max(0, i-size+1)..i and the blocks b whose last position b*pool+pool-1 <= i - size."""
    toks = list(range(max(0, i - size + 1), i + 1))
    blocks = [b for b in range(0, (i // pool) + 1) if b * pool + pool - 1 <= i - size]
    return toks, blocks


def window_pool_attention_mixer(h, pos, W: Dict[str, torch.Tensor], m: dict, eps: float, cache: dict,
                                cache_round=None):
    """Grouped-query attention over a sliding window plus one mean key / value per block of
    `pool` tokens that lies wholly before the window; weights are sigmoid(score + bias of the
    head), not normalised.  cache = {"k": [n, G, dk], "v": [n, G, dv]} of the earlier tokens (grows).
    cache_round: what the cache's storage does to a value (e.g. rounding to bfloat16)."""
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    size, P = m["mask"]["size"], m["mask"]["pool"]
    T = h.shape[0]
    rd = cache_round or (lambda t: t)
    q = (h @ W["q"].T).view(T, H, dk)
    k = (h @ W["k"].T).view(T, G, dk)
    v = (h @ W["v"].T).view(T, G, dv)
    q = unit_rms(rotate_interleaved_layout(q, pos, m["rot"]["dims"], m["rot"]["base"]), eps)
    k = unit_rms(rotate_interleaved_layout(k, pos, m["rot"]["dims"], m["rot"]["base"]), eps)
    cache["k"] = torch.cat([cache["k"], rd(k)]) if "k" in cache else rd(k)
    cache["v"] = torch.cat([cache["v"], rd(v)]) if "v" in cache else rd(v)
    K, V = cache["k"], cache["v"]
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for t in range(T):
        i = int(pos[t])
        toks, blocks = visible_keys(i, size, P)
        keys = [K[j] for j in toks] + [rd(K[b * P:(b + 1) * P].mean(0)) for b in blocks]
        vals = [V[j] for j in toks] + [rd(V[b * P:(b + 1) * P].mean(0)) for b in blocks]
        Kt, Vt = torch.stack(keys), torch.stack(vals)                      # [n, G, d]
        for hd in range(H):
            g = hd // (H // G)
            w = torch.sigmoid((Kt[:, g] @ q[t, hd]) * m["scale"] + W["pb"][hd])
            out[t, hd] = w @ Vt[:, g]
    gate = torch.sigmoid(h @ W["g"].T)
    return (out.reshape(T, H * dv) * gate) @ W["o"].T


def dense_ff(h, W: Dict[str, torch.Tensor]):
    return (torch.relu(h @ W["gate"].T) * (h @ W["up"].T)) @ W["down"].T


# ------------------------------------------------------------------ model
class Sequence:
    """What one sequence keeps between calls."""

    def __init__(self, cfg: dict, dtype=torch.float64):
        self.n = 0
        self.per_layer: List[object] = []
        for l in cfg["layers"]:
            m = l["mixer"]
            if l["type"] == "attention":
                self.per_layer.append({})
            else:
                self.per_layer.append(torch.zeros(m["heads"], m["dim"], m["vdim"], dtype=dtype))


def _sub(state: Dict[str, torch.Tensor], prefix: str, dtype) -> Dict[str, torch.Tensor]:
    return {k[len(prefix):]: t.to(dtype) for k, t in state.items() if k.startswith(prefix)}


def forward(cfg: dict, state: Dict[str, torch.Tensor], tokens: List[int], seq: Sequence,
            dtype=torch.float64, cache_round=None, layer_outputs: Optional[list] = None) -> torch.Tensor:
    """Feeds `tokens` as the next tokens of `seq`; returns the logits of each, [T, vocab]."""
    eps = cfg["norm"]["eps"]
    pos = torch.arange(seq.n, seq.n + len(tokens))
    emb = state["embed"].to(dtype)
    x = emb[torch.tensor(tokens)]
    for i, l in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = offset_rms_norm(x, state[p + "norm1"].to(dtype), eps)
        Wm = _sub(state, p + "mix.", dtype)
        fn = {"retention": retention_mixer, "gla": gla_mixer}.get(l["type"])
        if fn is not None:
            y = fn(h, pos, Wm, l["mixer"], eps, seq.per_layer[i])
        elif l["type"] == "attention":
            y = window_pool_attention_mixer(h, pos, Wm, l["mixer"], eps, seq.per_layer[i], cache_round)
        else:
            raise ValueError(l["type"])
        r1 = torch.sigmoid(h @ state[p + "rg1"].to(dtype).T + state[p + "rg1.b"].to(dtype))
        x_new = x + r1 * y
        if l.get("mlp"):
            r2 = torch.sigmoid(h @ state[p + "rg2"].to(dtype).T + state[p + "rg2.b"].to(dtype))
            x_new = x_new + r2 * dense_ff(h, _sub(state, p + "mlp.", dtype))
        x = x_new
        if layer_outputs is not None:
            layer_outputs.append(x.clone())
    seq.n += len(tokens)
    return offset_rms_norm(x, state["final.norm"].to(dtype), eps) @ emb.T


# ------------------------------------------------------------------ random models for tests
def random_model(cfg: dict, seed: int = 0, scale: float = 1.0) -> Dict[str, torch.Tensor]:
    """Seeded random tensors under the checkpoint's names, rounded to bfloat16 values (float32
    storage), sized so that activations stay of order one."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def rn(*shape, s):
        return (torch.randn(*shape, generator=g) * s * scale).to(torch.bfloat16).float()

    st = {"embed": rn(cfg["vocab"], W, s=1.0), "final.norm": rn(W, s=0.1)}
    for i, l in enumerate(cfg["layers"]):
        p, m = f"l{i}.", l["mixer"]
        H, dk, dv = m["heads"], m["dim"], m["vdim"]
        G = m.get("kv_heads", H)
        st[p + "norm1"] = rn(W, s=0.1)
        st[p + "mix.q"] = rn(H * dk, W, s=W ** -0.5)
        st[p + "mix.k"] = rn(G * dk, W, s=W ** -0.5)
        st[p + "mix.v"] = rn(G * dv, W, s=W ** -0.5)
        st[p + "mix.g"] = rn(H * dv, W, s=W ** -0.5)
        st[p + "mix.o"] = rn(W, H * dv, s=(H * dv) ** -0.5)
        if l["type"] == "attention":
            st[p + "mix.pb"] = rn(H, s=1.0) - 2.0
        if l["type"] == "gla":
            r = m.get("rank", 8)
            st[p + "mix.norm"] = 1 + rn(dv, s=0.1)
            st[p + "mix.a1"] = rn(r, W, s=W ** -0.5)
            st[p + "mix.a2"] = rn(H * dk, r, s=r ** -0.5)
            st[p + "mix.a2.b"] = rn(H * dk, s=1.0) + 3.0
        st[p + "rg1"] = rn(W, W, s=W ** -0.5)
        st[p + "rg1.b"] = rn(W, s=0.5)
        if l.get("mlp"):
            F = l["mlp"]["ff"]
            st[p + "mlp.gate"] = rn(F, W, s=W ** -0.5)
            st[p + "mlp.up"] = rn(F, W, s=W ** -0.5)
            st[p + "mlp.down"] = rn(W, F, s=F ** -0.5)
            st[p + "rg2"] = rn(W, W, s=W ** -0.5)
            st[p + "rg2.b"] = rn(W, s=0.5)
    return st
