"""A plain, slow implementation of the Sovutar decoder in PyTorch on the CPU, one function per
mechanism, written from the design's equations.  It shares no code with the engine: it reads
config.json as a dictionary and the tensors by name, and keeps nothing between calls.

Notation: T tokens, W model width.  A layer is x <- x + N1(mixer(x)), x <- x + N2(ff(x)) with
N(y) = y / rms(y) * (1 + w): the norm sits on the sublayer's output, the sublayers read x itself.
Mixers: a chunked grouped-query attention without positions whose q and k are normed over the whole
projection and whose values may be mixed with those of the first such layer; a latent attention
(one compressed key/value vector a token, one rotated key part shared by the heads) over a sliding
window with a sink in the softmax's denominator.  The feed-forward is a mixture of experts with a
sigmoid router and a shared expert.  The logits are soft-capped.
"""
from __future__ import annotations

import math

import torch


def rms_unit(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def one_plus_norm(x, w, eps):
    """RMS norm with a weight stored around zero."""
    return rms_unit(x, eps) * (1.0 + w)


def rotate_interleaved(x, positions, base, dims):
    """Rotary encoding of the first `dims` entries of the last axis of x [T, ..., D]: entry 2i is paired with
    2i + 1, the angle at position p is p * base^(-2i/dims)."""
    T = x.shape[0]
    half = dims // 2
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=x.dtype)
    angle = positions.to(x.dtype)[:, None] * freq[None, :]                 # [T, half]
    shape = [T] + [1] * (x.dim() - 2) + [half]
    cos, sin = torch.cos(angle).view(shape), torch.sin(angle).view(shape)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * cos - v * sin
    out[..., 1:dims:2] = v * cos + u * sin
    return out


def softmax_attention(scores, visible, values, sink=None):
    """scores [H, T, T] (row i, key j), visible bool [T, T], values [H, T, Dv]; sink [H] or None: an extra
    term exp(sink_h) in the denominator that has no value."""
    s = scores.masked_fill(~visible[None], float("-inf"))
    m = s.max(-1, keepdim=True).values
    if sink is not None:
        m = torch.maximum(m, sink[:, None, None])
    e = torch.exp(s - m)
    denom = e.sum(-1, keepdim=True)
    if sink is not None:
        denom = denom + torch.exp(sink[:, None, None] - m)
    return (e / denom) @ values


def window_mask(T, size):
    """Row i sees j with 0 <= i - j < size (size None: every j <= i)."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    seen = j <= i
    if size is not None:
        seen &= (i - j) < size
    return seen


def chunk_mask(T, size):
    """Row i sees j <= i in its own chunk of `size` positions, counted from position 0 (size None: every j <= i)."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    seen = j <= i
    if size is not None:
        seen &= (i // size) == (j // size)
    return seen


def chunked_attention(h, p, m, eps, v_first):
    """The 'attention' mixer.  Returns (output [T, W], the values of this layer before mixing [T, G * Dv]).
    v_first: the values of the first value-mixing layer, or None if this layer is that one or does not mix."""
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = rms_unit(h @ p["q"].T, eps) * p["q.norm"]          # over the whole projection, plain weights
    k = rms_unit(h @ p["k"].T, eps) * p["k.norm"]
    v_own = h @ p["v"].T
    v = v_own
    if v_first is not None:
        lam = p["vmix"]
        v = (1.0 - lam) * v_own + lam * v_first
    q = q.view(T, H, D).transpose(0, 1)                       # [H, T, D]
    k = k.view(T, G, D).transpose(0, 1).repeat_interleave(H // G, dim=0)
    vv = v.view(T, G, Dv).transpose(0, 1).repeat_interleave(H // G, dim=0)
    scores = (q @ k.transpose(1, 2)) * m["scale"]
    size = m["mask"]["size"] if m.get("mask") else None
    out = softmax_attention(scores, chunk_mask(T, size), vv)
    return out.transpose(0, 1).reshape(T, H * Dv) @ p["o"].T, v_own


def latent_attention(h, p, m, eps):
    """The 'latent_attention' mixer, in the form that expands keys and values of every token."""
    H, D, R, Dv, C = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    T = h.shape[0]
    pos = torch.arange(T)
    q = (h @ p["q"].T).view(T, H, D + R)
    q_plain, q_rot = q[..., :D], q[..., D:]
    down = h @ p["dkv"].T
    c = rms_unit(down[:, :C], eps) * p["dkv.norm"]
    k_rot = down[:, C:]
    base, dims = m["rot"]["base"], m["rot"]["dims"]
    q_rot = rotate_interleaved(q_rot, pos, base, dims)
    k_rot = rotate_interleaved(k_rot, pos, base, dims)
    k_plain = (c @ p["uk"].T).view(T, H, D)
    v = (c @ p["uv"].T).view(T, H, Dv)
    scores = (torch.einsum("ihd,jhd->hij", q_plain, k_plain) + torch.einsum("ihr,jr->hij", q_rot, k_rot)) * m["scale"]
    size = m["mask"]["size"] if m.get("mask") else None
    out = softmax_attention(scores, window_mask(T, size), v.transpose(0, 1), sink=p["sink"])
    return out.transpose(0, 1).reshape(T, H * Dv) @ p["o"].T


def silu(z):
    return z * torch.sigmoid(z)


def expert(h, p, prefix):
    return (silu(h @ p[prefix + "gate"].T) * (h @ p[prefix + "up"].T)) @ p[prefix + "down"].T


def moe(h, p, mlp):
    """Sigmoid router; the experts are chosen by score + correction, weighted by their scores alone."""
    r = mlp["router"]
    E, top = r["experts"], r["top"]
    s = torch.sigmoid(h @ p["router"].T)                      # [T, E]
    chosen = torch.topk(s + p["correction"], top, dim=-1).indices
    w = torch.gather(s, 1, chosen)
    w = w / (w.sum(-1, keepdim=True) + 1e-20) * r["scale"]
    out = torch.zeros_like(h)
    for e in range(E):
        y = expert(h, p, f"e{e}.")
        weight = (w * (chosen == e)).sum(-1, keepdim=True)     # zero where the expert was not chosen
        out = out + weight * y
    if mlp.get("shared") is not None:
        out = out + expert(h, p, "shared.")
    return out


def forward(config: dict, tensors: dict, tokens, dtype=torch.float64, layers_out: list | None = None):
    """Logits [T, vocab] of one sequence from position 0.  layers_out: a list that receives the residual stream
    after every layer."""
    t = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in tensors.items()}
    eps = config["norm"]["eps"]
    x = t["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    v_first = None
    for i, layer in enumerate(config["layers"]):
        sub = lambda part: {k[len(f"l{i}.{part}."):]: v for k, v in t.items() if k.startswith(f"l{i}.{part}.")}
        m = layer["mixer"]
        if layer["type"] == "attention":
            mixes = bool(m.get("v_mix"))
            y, v_own = chunked_attention(x, sub("mix"), m, eps, v_first if mixes else None)
            if mixes and v_first is None:
                v_first = v_own
        elif layer["type"] == "latent_attention":
            y = latent_attention(x, sub("mix"), m, eps)
        else:
            raise ValueError(layer["type"])
        x = x + one_plus_norm(y, t[f"l{i}.norm1"], eps)
        if layer.get("mlp") is not None:
            x = x + one_plus_norm(moe(x, sub("mlp"), layer["mlp"]), t[f"l{i}.norm2"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    z = one_plus_norm(x, t["final.norm"], eps) @ t["head"].T
    cap = config.get("logit_softcap")
    return cap * torch.tanh(z / cap) if cap else z
