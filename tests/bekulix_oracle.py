"""Plain, slow oracle of the Bekulix design for the tests: one function per
mechanism, written from the design's equations with dense [T, T] masks and
whole sequences, float64 throughout.  It shares nothing with the engine's
model, ops or kernels; it only consumes a config dict and a name -> tensor
dict in the checkpoint's own naming.

Notation: T tokens of one sequence at positions 0 .. T-1, h the mixer input
[T, width], weights stored [out, in] and applied as h @ W^T.
"""
from __future__ import annotations

import math

import torch

F = torch.float64


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_one_plus(x, w, eps):
    """Layer / final norm: unit RMS times (1 + w)."""
    return rms(x, eps) * (1.0 + w)


def norm_plain(x, w, eps):
    return rms(x, eps) * w


def visible(T: int, kind: str, size: int | None) -> torch.Tensor:
    """[T, T] bool, row i column j: may query i see key j."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    m = j <= i
    if kind == "window":
        m &= (i - j) < size
    elif kind == "chunk":
        m &= (i // size) == (j // size)
    elif kind != "causal":
        raise ValueError(kind)
    return m


def softmax_attend(q, k, v, scale, mask):
    """q [T, H, d], k [T, H, d], v [T, H, dv] (key heads already expanded)."""
    s = torch.einsum("ihd,jhd->hij", q, k) * scale
    s = s.masked_fill(~mask[None], float("-inf"))
    p = torch.softmax(s, dim=-1)
    return torch.einsum("hij,jhd->ihd", p, v)


def expand_heads(x, H):
    """[T, G, d] -> [T, H, d]: query head h reads group h // (H / G)."""
    G = x.shape[1]
    return x.repeat_interleave(H // G, dim=1)


def mixer_attention(h, W, pre, m, eps):
    T = h.shape[0]
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    q = (h @ W[pre + "q"].T).view(T, H, d)
    k = (h @ W[pre + "k"].T).view(T, G, d)
    v = k  # the values are the keys as projected
    q = norm_plain(q, W[pre + "q.norm"], eps)
    kn = norm_plain(k, W[pre + "k.norm"], eps)
    qt = m.get("q_temp")
    if qt:
        p = torch.arange(T, dtype=F)
        f = 1.0 + qt["coef"] * torch.log(torch.floor((p + 1) / qt["every"]) + 1.0)
        q = q * f[:, None, None]
    o = softmax_attend(q, expand_heads(kn, H), expand_heads(v, H), m["scale"], visible(T, "causal", None))
    return o.reshape(T, -1) @ W[pre + "o"].T


def mixer_latent(h, W, pre, m, eps):
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ W[pre + "q"].T).view(T, H, d)
    c = norm_plain(h @ W[pre + "dkv"].T, W[pre + "dkv.norm"], eps)
    k = (c @ W[pre + "uk"].T).view(T, H, d)
    v = (c @ W[pre + "uv"].T).view(T, H, dv)
    o = softmax_attend(q, k, v, m["scale"], visible(T, "window", m["mask"]["size"]))
    return o.reshape(T, -1) @ W[pre + "o"].T


def mixer_differential(h, W, pre, m, eps):
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ W[pre + "q"].T + W[pre + "q.b"]).view(T, H, 2, d)
    k = (h @ W[pre + "k"].T + W[pre + "k.b"]).view(T, G, 2, d)
    v = (h @ W[pre + "v"].T + W[pre + "v.b"]).view(T, G, dv)
    mask = visible(T, "chunk", m["mask"]["size"])
    ve = expand_heads(v, H)
    a = [softmax_attend(q[:, :, i], expand_heads(k[:, :, i], H), ve, m["scale"], mask) for i in range(2)]
    diff = m["diff"]
    lam = math.exp(float((W[pre + "lq1"] * W[pre + "lk1"]).sum())) \
        - math.exp(float((W[pre + "lq2"] * W[pre + "lk2"]).sum())) + diff
    o = rms(a[0] - lam * a[1], eps) * (1.0 - diff)
    return o.reshape(T, -1) @ W[pre + "o"].T


MIXERS = {"attention": mixer_attention, "latent_attention": mixer_latent, "attention_2": mixer_differential}


def feed_forward(h, W, pre, mlp):
    if mlp["kind"] != "dense":
        raise ValueError(mlp["kind"])
    return (torch.relu(h @ W[pre + "gate"].T) * (h @ W[pre + "up"].T)) @ W[pre + "down"].T


def hyper_sublayer(xs, W, pre, fn, norm_w, eps):
    """xs [S, T, width]; one sublayer under hyper-connections."""
    u = torch.einsum("s,stw->tw", W[pre + "in"], xs)
    y = fn(norm_one_plus(u, norm_w, eps))
    return torch.einsum("st,sjw->tjw", W[pre + "mix"], xs) + W[pre + "out"][:, None, None] * y[None]


def layer_schedule(cfg) -> list[int]:
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp:
        return list(range(n))
    body = list(range(lp["start"], lp["stop"]))
    return list(range(lp["start"])) + body * lp["times"] + list(range(lp["stop"], n))


def forward(cfg: dict, weights: dict, tokens: list[int], return_layers: bool = False):
    """Logits [T, vocab] of one whole sequence (and the residual stream after
    every layer run when asked)."""
    W = {k: v.to(F) for k, v in weights.items() if v.dtype != torch.int32}
    eps = cfg["norm"]["eps"]
    S = cfg.get("streams")
    x = W["embed"][torch.tensor(tokens)]
    xs = x[None].repeat(S, 1, 1) if S else None
    trail = []
    for li in layer_schedule(cfg):
        spec = cfg["layers"][li]
        pre = f"l{li}."
        mix = lambda z: MIXERS[spec["type"]](z, W, pre + "mix.", spec["mixer"], eps)  # noqa: E731
        ff = (lambda z: feed_forward(z, W, pre + "mlp.", spec["mlp"])) if spec.get("mlp") else None
        if S:
            xs = hyper_sublayer(xs, W, pre + "hc1.", mix, W[pre + "norm1"], eps)
            if ff:
                xs = hyper_sublayer(xs, W, pre + "hc2.", ff, W[pre + "norm2"], eps)
            trail.append(xs.sum(0))
        else:
            x = x + mix(norm_one_plus(x, W[pre + "norm1"], eps))
            if ff:
                x = x + ff(norm_one_plus(x, W[pre + "norm2"], eps))
            trail.append(x)
    if S:
        x = xs.sum(0)
    logits = norm_one_plus(x, W["final.norm"], eps) @ W["head"].T
    return (logits, torch.stack(trail)) if return_layers else logits
