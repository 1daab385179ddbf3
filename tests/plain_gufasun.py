"""A plain, slow implementation of the Gufasun decoder in PyTorch on the CPU, one function per
mechanism, written from the design's equations.  It shares no code with the engine: it reads
config.json as a dictionary and the tensors by name, walks every sequence token by token where
the design is recurrent, and keeps nothing between calls.

Notation: T tokens, W model width, per layer a mixer (windowed attention or an mLSTM matrix
memory) and a feed-forward that both read the same residual x (two layer norms), whose outputs
are added to x together.  What the mixer reads first passes h <- h + causal_conv(h).
"""
from __future__ import annotations

import torch


def layer_norm(x, w, eps):
    """(x - mean) / sqrt(var + eps) * w, var = mean of squared deviations; no bias."""
    mu = x.mean(-1, keepdim=True)
    d = x - mu
    return d / torch.sqrt((d * d).mean(-1, keepdim=True) + eps) * w


def rms_unit(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def causal_conv(u, w):
    """y_t = sum_j w[:, j] u_(t - taps + 1 + j) over time for u [T, C], w [C, taps]; zeros before the start."""
    T, C = u.shape
    taps = w.shape[1]
    y = torch.zeros_like(u)
    for j in range(taps):
        back = taps - 1 - j
        if back < T:
            y[back:] += w[:, j] * u[:T - back]
    return y


def poly_norm_ffn(h, up, up_b, down, down_b, coef, eps):
    """down(a N(z) + b N(z^2) + c N(z^3) + e) + bias with z = up h + bias, N = division by the row's rms."""
    z = h @ up.T + up_b
    a, b, c, e = [coef[i] for i in range(4)]
    act = a * rms_unit(z, eps) + b * rms_unit(z * z, eps) + c * rms_unit(z * z * z, eps) + e
    return act @ down.T + down_b


def attention_keys_values(h, p, m, eps):
    """Keys (after convolution and norm) and values (after convolution) of one layer for h [T, W]."""
    G, D, Dv = m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    k, v = h @ p["k"].T + p["k.b"], h @ p["v"].T + p["v.b"]
    if m.get("conv"):
        k, v = causal_conv(k, p["k.conv"]), causal_conv(v, p["v.conv"])
    k = rms_unit(k.view(T, G, D), eps) * p["k.norm"]
    return k, v.view(T, G, Dv)


def attention_mixer(h, p, m, eps, keys, values):
    """Windowed soft-capped attention with a logarithmic distance penalty; keys [T, G, D], values [T, G, Dv]."""
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    T = h.shape[0]
    q = h @ p["q"].T + p["q.b"]
    if m.get("conv"):
        q = causal_conv(q, p["q.conv"])
    q = rms_unit(q.view(T, H, D), eps) * p["q.norm"]
    pos = torch.arange(T, dtype=h.dtype)
    if m.get("q_temp"):
        temp = 1 + m["q_temp"]["coef"] * torch.log(torch.floor((pos + 1) / m["q_temp"]["every"]) + 1)
        q = q * temp[:, None, None]
    cap, window = m.get("softcap", 0.0), m["mask"]["size"]
    out = torch.zeros(T, H, values.shape[-1], dtype=h.dtype)
    for hq in range(H):
        g = hq // (H // G)
        for i in range(T):
            lo = max(0, i - window + 1)
            s = (keys[lo:i + 1, g] @ q[i, hq]) * m["scale"]
            if cap:
                s = cap * torch.tanh(s / cap)
            dist = (i - torch.arange(lo, i + 1)).to(h.dtype)
            s = s - p["r1"][hq] * torch.log1p(p["r2"][hq] * dist)
            out[i, hq] = torch.softmax(s, 0) @ values[lo:i + 1, g]
    return out.reshape(T, -1) @ p["o"].T


def mlstm_mixer(h, p, m, eps):
    """Matrix memory with exponential gates and a running maximum m that starts at 0, token by token."""
    H, D, Dv, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    T = h.shape[0]
    q = (h @ p["q"].T).view(T, H, D) * D ** -0.5
    k = (h @ p["k"].T).view(T, H, D)
    v = (h @ p["v"].T).view(T, H, Dv)
    gi = cap * torch.tanh((h @ p["i"].T + p["i.b"]) / cap)
    gf = torch.nn.functional.logsigmoid(cap * torch.tanh((h @ p["f"].T + p["f.b"]) / cap))
    S = torch.zeros(H, D, Dv, dtype=h.dtype)
    n = torch.zeros(H, D, dtype=h.dtype)
    mx = torch.zeros(H, dtype=h.dtype)
    out = torch.zeros(T, H, Dv, dtype=h.dtype)
    for t in range(T):
        m_new = torch.maximum(gf[t] + mx, gi[t])
        keep = torch.exp(gf[t] + mx - m_new)
        take = torch.exp(gi[t] - m_new)
        S = keep[:, None, None] * S + take[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = keep[:, None] * n + take[:, None] * k[t]
        mx = m_new
        num = torch.einsum("hdv,hd->hv", S, q[t])
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-mx)) + 1e-6
        out[t] = num / den[:, None]
    out = rms_unit(out, eps).reshape(T, -1) * p["norm"]
    out = out * torch.sigmoid(h @ p["g"].T)
    return out @ p["o"].T


def _sub(weights, prefix):
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def forward(weights, cfg, tokens, dtype=torch.float64, return_layers=False):
    """Logits [T, vocab] of one whole sequence (and the residual stream after every layer if asked)."""
    W = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.tensor(tokens, dtype=torch.long)] * cfg["embedding"]["scale"]
    kept, trail = {}, []
    for i, layer in enumerate(cfg["layers"]):
        p = _sub(W, f"l{i}.")
        h = layer_norm(x, p["norm1"], eps)
        h = h + causal_conv(h, p["canon1"])
        mp, m = _sub(p, "mix."), layer["mixer"]
        if layer["type"] == "attention":
            if m.get("kv_from") is None:
                kept[i] = attention_keys_values(h, mp, m, eps)
            keys, values = kept[m["kv_from"] if m.get("kv_from") is not None else i]
            mixed = attention_mixer(h, mp, m, eps, keys, values)
        elif layer["type"] == "mlstm":
            mixed = mlstm_mixer(h, mp, m, eps)
        else:
            raise ValueError(f"unknown layer type {layer['type']!r}")
        if layer.get("mlp") is not None:
            f = _sub(p, "mlp.")
            mixed = mixed + poly_norm_ffn(layer_norm(x, p["norm2"], eps), f["up"], f["up.b"], f["down"], f["down.b"],
                                          f["act"], eps)
        x = x + mixed
        trail.append(x)
    logits = layer_norm(x, W["final.norm"], eps) @ W["head"].T
    return (logits, torch.stack(trail)) if return_layers else logits


def forward_logits(weights, cfg, tokens, dtype=torch.float64):
    return forward(weights, cfg, tokens, dtype=dtype)
