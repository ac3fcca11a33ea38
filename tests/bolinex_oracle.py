"""Plain, slow oracle of the Bolinex design for the tests: one function per
mechanism, dense [T, T] score matrices over whole sequences, float64
throughout.  It shares nothing with the engine's model, ops or kernels; it
consumes a config dict (the keys of a checkpoint's config.json) and a
name -> tensor dict in the checkpoint's naming.

Notation: T tokens of one sequence at positions 0 .. T-1; x [T, width] the
residual; h the normed sublayer input; weights stored [out, in], applied as
h @ W^T.
"""
from __future__ import annotations

import math

import torch

F = torch.float64


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def layer_norm(x, w, b, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def embed(W, toks):
    """Token rows plus the learned vector of each position."""
    T = len(toks)
    return W["embed"][toks] + W["pos"][:T]


def window_mask(T, size):
    """[T, T] bool: query i sees key j when 0 <= i - j < size (size None: every earlier key)."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    m = j <= i
    if size is not None:
        m &= (i - j) < size
    return m


def scores(q, k, scale, softcap, r1, r2):
    """[H, T, T] scores before the mask: scaled products, tanh cap, then the
    distance penalty r1_h ln(1 + r2_h (i - j)) taken off.  q, k [T, H, d]."""
    T = q.shape[0]
    s = torch.einsum("ihd,jhd->hij", q, k) * scale
    if softcap:
        s = softcap * torch.tanh(s / softcap)
    if r1 is not None:
        dist = (torch.arange(T)[:, None] - torch.arange(T)[None, :]).clamp_min(0).to(F)
        s = s - r1[:, None, None] * torch.log(1.0 + r2[:, None, None] * dist[None])
    return s


def attend(s, v, mask):
    """softmax over the visible keys, weighted sum of v [T, H, dv] -> [T, H, dv]."""
    p = torch.softmax(s.masked_fill(~mask[None], float("-inf")), dim=-1)
    return torch.einsum("hij,jhd->ihd", p, v)


def value_mix(v, v_first, lam):
    return (1.0 - lam) * v + lam * v_first


def mixer_attention(h, W, pre, m, v_first):
    """Returns (mixer output [T, width], this layer's values as projected)."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ W[pre + "q"].T).view(T, H, d)
    k = (h @ W[pre + "k"].T).view(T, G, d)
    v_own = (h @ W[pre + "v"].T).view(T, G, dv)
    v = v_own
    if m.get("v_mix") and v_first is not None:
        v = value_mix(v_own, v_first, W[pre + "vmix"])
    rep = H // G
    s = scores(q, k.repeat_interleave(rep, 1), m["scale"], m.get("softcap"), W.get(pre + "r1"), W.get(pre + "r2"))
    size = (m.get("mask") or {}).get("size")
    a = attend(s, v.repeat_interleave(rep, 1), window_mask(T, size)).reshape(T, H * dv)
    if pre + "g" in W:
        a = a * torch.sigmoid(h @ W[pre + "g"].T)
    return a @ W[pre + "o"].T, v_own


def ff_dense(h, W, pre):
    return torch.relu(h @ W[pre + "up"].T) ** 2 @ W[pre + "down"].T


def expert(h, W, pre):
    g = h @ W[pre + "gate"].T
    return (g * torch.sigmoid(g) * (h @ W[pre + "up"].T)) @ W[pre + "down"].T


def route(z, correction, top, groups, margin=None):
    """Per token: chosen experts [T, top] and their weights.  z [T, E] router logits.
    margin (a list): gets a [T] tensor, how far each token's choice is from another one
    (the gap between the last score taken and the first one left, of groups and of experts)."""
    s = torch.sigmoid(z)
    c = s + correction
    T, E = c.shape
    gap = torch.full((T,), float("inf"), dtype=c.dtype)
    if groups:
        n, keep = groups["count"], groups["keep"]
        per = E // n
        cg = c.view(T, n, per)
        gs = cg.topk(min(2, per), -1).values.sum(-1)
        kept = torch.zeros(T, n, dtype=torch.bool)
        kept.scatter_(1, gs.topk(keep, -1).indices, True)
        if keep < n:
            g = gs.sort(-1, descending=True).values
            gap = g[:, keep - 1] - g[:, keep]
        c = c.masked_fill(~kept[:, :, None].expand(T, n, per).reshape(T, E), float("-inf"))
    idx = c.topk(top, -1).indices
    if top < E:
        cs = c.sort(-1, descending=True).values
        gap = torch.minimum(gap, cs[:, top - 1] - cs[:, top])
    if margin is not None:
        margin.append(gap)
    return idx, s.gather(1, idx)


def ff_moe(h, W, pre, mlp, margin=None):
    r = mlp["router"]
    idx, wgt = route(h @ W[pre + "router"].T, W[pre + "correction"], r["top"], r.get("groups"), margin)
    out = torch.zeros(h.shape[0], W[pre + "e0.down"].shape[0], dtype=F)
    for t in range(h.shape[0]):
        for e, w in zip(idx[t].tolist(), wgt[t]):
            out[t] += w * expert(h[t:t + 1], W, f"{pre}e{e}.")[0]
    if mlp.get("shared"):
        out = out + expert(h, W, pre + "shared.")
    return out


def token_side(x, W, i, toks, dim, eps):
    """The per-layer token input of layer i, added to the residual."""
    e = W["side.embed"][toks][:, i * dim:(i + 1) * dim]
    g = gelu_tanh(x @ W[f"l{i}.side.gate"].T) * e
    y = g @ W[f"l{i}.side.proj"].T
    return x + unit_rms(y, eps) * W[f"l{i}.side.norm"]


def forward(cfg: dict, W: dict, toks, return_layers: bool = False, margin: list | None = None):
    W = {k: (v.to(F) if v.is_floating_point() else v) for k, v in W.items()}
    eps = cfg["norm"]["eps"]
    toks = torch.as_tensor(toks, dtype=torch.long)
    x = embed(W, toks)
    v_first = None
    layers = []
    for i, L in enumerate(cfg["layers"]):
        h = layer_norm(x, W[f"l{i}.norm1"], W[f"l{i}.norm1.b"], eps)
        y, v_own = mixer_attention(h, W, f"l{i}.mix.", L["mixer"], v_first)
        if L["mixer"].get("v_mix") and v_first is None:
            v_first = v_own
        mlp = L.get("mlp")
        if mlp:
            y = y + (ff_dense(h, W, f"l{i}.mlp.") if mlp["kind"] == "dense" else ff_moe(h, W, f"l{i}.mlp.", mlp, margin))
        x = x + y
        if cfg.get("token_side"):
            x = token_side(x, W, i, toks, cfg["token_side"]["dim"], eps)
        layers.append(x)
    logits = layer_norm(x, W["final.norm"], W["final.norm.b"], eps) @ W["head"].T
    return (logits, torch.stack(layers)) if return_layers else logits
