"""Tiny Sovutar configurations for tests, and helpers that make model folders from them.

P: chunked attention (the source of mixed values), latent attention, a chunked attention that mixes, a latent one
again; key and value sizes differ everywhere, three q heads a kv head, five experts of which two are chosen.
Q: what models often make equal differs and what is often large is 1: a latent layer first, a chunked layer that does
not mix, one that would be the source with nobody mixing, a layer without feed-forward, one choice of three experts, no
shared expert, a chunk of one page, a window of one key, one head, rotary dims below the rotated part's size.
R: sizes the matrix-core attention takes (keys of 64 and of 96 + 32, values of 64 and 96), windows and chunks of
several pages, every expert chosen (no close call in the router, whatever the precision).
S: sizes it does not take (a key size that is a multiple of 8 only, a value size that is no multiple of 16), five q
heads on one kv head, seventy experts of which three are chosen, no logit cap.
"""
from __future__ import annotations

import os

import torch
from safetensors.torch import load_file, save_file

from arle_amd.config import SovutarConfig
from arle_amd.weights import write_random_model

ARCH = "Sovutar"


def chunked(heads, kv_heads, dim, vdim, chunk, v_mix=True, scale=0.3):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "v_mix": v_mix}
    if chunk is not None:
        m["mask"] = {"size": chunk}
    return m


def latent(heads, dim, rot_dim, vdim, rank, window, scale=0.2, base=10000.0, dims=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank, "scale": scale,
         "rot": {"base": base, "dims": rot_dim if dims is None else dims}}
    if window is not None:
        m["mask"] = {"size": window}
    return m


def moe(experts, top, ff, shared, scale=2.0):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "scale": scale},
            "shared": None if shared is None else {"ff": shared}}


def layer(kind, mixer, mlp):
    return {"type": kind, "mixer": mixer, "mlp": mlp}


TINY_P = {"architecture": ARCH, "vocab": 211, "width": 72, "norm": {"eps": 2e-5}, "logit_softcap": 8.0,
          "layers": [layer("attention", chunked(6, 2, 16, 24, chunk=11), moe(5, 2, 40, 56)),
                     layer("latent_attention", latent(3, 24, 8, 20, 40, window=9), moe(5, 2, 40, 56)),
                     layer("attention", chunked(6, 2, 16, 24, chunk=30, scale=0.5), moe(4, 3, 24, 32, scale=1.0)),
                     layer("latent_attention", latent(4, 16, 16, 12, 32, window=26, base=500.0), moe(5, 2, 40, 56))]}

TINY_Q = {"architecture": ARCH, "vocab": 97, "width": 40, "norm": {"eps": 1e-6}, "logit_softcap": 30.0,
          "layers": [layer("latent_attention", latent(1, 8, 12, 16, 24, window=1, dims=6), moe(3, 1, 16, None)),
                     layer("attention", chunked(2, 2, 32, 8, chunk=8, v_mix=False), None),
                     layer("attention", chunked(4, 1, 8, 16, chunk=None), moe(3, 1, 16, None, scale=0.7)),
                     layer("latent_attention", latent(2, 8, 4, 8, 16, window=None), moe(2, 2, 8, 24))]}

TINY_R = {"architecture": ARCH, "vocab": 300, "width": 96, "norm": {"eps": 1e-5}, "logit_softcap": 12.0,
          "layers": [layer("attention", chunked(4, 2, 64, 64, chunk=40), moe(3, 3, 48, 64)),
                     layer("attention", chunked(4, 2, 32, 64, chunk=50, scale=0.4), moe(2, 2, 32, 48)),
                     layer("latent_attention", latent(4, 32, 32, 32, 96, window=37), moe(3, 3, 48, 64)),
                     layer("latent_attention", latent(20, 16, 16, 16, 48, window=70, base=250000.0), moe(4, 4, 16, 16))]}

TINY_S = {"architecture": ARCH, "vocab": 150, "width": 60, "norm": {"eps": 1e-5},
          "layers": [layer("latent_attention", latent(5, 12, 8, 28, 72, window=19), moe(70, 3, 12, 20)),
                     layer("attention", chunked(5, 1, 24, 40, chunk=21), moe(6, 5, 20, 12)),
                     layer("attention", chunked(5, 1, 24, 40, chunk=64, scale=0.2), None)]}

# name -> (config, page size, weight std, norm std, seed)
TINY = {"P": (TINY_P, 4, 0.15, 0.2, 5), "Q": (TINY_Q, 8, 0.2, 0.3, 6), "R": (TINY_R, 16, 0.1, 0.2, 7),
        "S": (TINY_S, 16, 0.2, 0.2, 9)}
# the configurations whose routers choose every expert: their logits cannot hang on a close call in any precision
NO_CLOSE_CALLS = ("R",)


def make_model_dir(tmp_path, name: str) -> str:
    raw, _, std, norm_std, seed = TINY[name]
    d = os.path.join(str(tmp_path), f"sovutar_{name}")
    write_random_model(d, ARCH, SovutarConfig.from_dict(raw), seed=seed, std=std, norm_std=norm_std)
    # Constants as a trained model may have them, large enough that leaving one out shows: mixing weights of a few
    # tenths, sinks of the size of the scores, corrections that change who is chosen.
    path = os.path.join(d, "model.safetensors")
    tensors = load_file(path)
    g = torch.Generator().manual_seed(seed)
    for key, t in tensors.items():
        if key.endswith(".mix.vmix"):
            tensors[key] = torch.tensor(0.2 + 0.5 * float(torch.rand((), generator=g))).to(t.dtype)
        elif key.endswith(".mix.sink"):
            tensors[key] = (torch.randn(t.shape, generator=g) + 1.0).to(t.dtype)
        elif key.endswith(".mlp.correction"):
            tensors[key] = (torch.randn(t.shape, generator=g) * 0.3).to(t.dtype)
        elif key.endswith(".mlp.router"):
            tensors[key] = (t.float() * 4.0).to(t.dtype)
    save_file(tensors, path)
    return d
