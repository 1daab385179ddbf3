"""Tiny Gufasun configurations for tests, and helpers that make model folders from them.

P: four layers in the order attention, mlstm, attention that reads the first one's keys and values through a wider
window, mlstm without a feed-forward; key and value sizes differ everywhere, three q heads a kv head.
Q: the values that often coincide are made to differ, and the ones that are often large are 1: one tap in the input
convolution, one kv head a q head, a window of one page and one of a single key, a temperature period of 1, one
mLSTM head, no convolution on q, k and v in one layer, a value size that is no multiple of 16.
R: wider heads (a key size over 64, a value size over 64 that is no multiple of 64) and windows of several pages.
S: nothing but matrix memories (no paged cache at all).  T: nothing but attention, five q heads a kv head, a key size
that is a multiple of 8 only, a reader right behind its owner, and no feed-forward anywhere.
"""
from __future__ import annotations

import os

from safetensors.torch import load_file, save_file

from arle_amd.config import GufasunConfig
from arle_amd.weights import write_random_model

ARCH = "Gufasun"


def attention(heads, kv_heads, dim, vdim, window, conv=3, scale=0.25, softcap=6.0, coef=0.4, every=3, kv_from=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "softcap": softcap, "conv": conv,
         "mask": {"size": window}, "q_temp": {"coef": coef, "every": every}}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def mlstm(heads, dim, vdim, cap=9.0):
    return {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}


def layer(kind, mixer, ff):
    return {"type": kind, "mixer": mixer, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


TINY_P = {"architecture": ARCH, "vocab": 211, "width": 72, "norm": {"eps": 2e-5}, "embedding": {"scale": 5.5},
          "canon": {"taps": 3},
          "layers": [layer("attention", attention(6, 2, 16, 32, window=7), 100),
                     layer("mlstm", mlstm(3, 12, 20), 88),
                     layer("attention", attention(6, 2, 16, 32, window=21, softcap=3.0, every=5, kv_from=0), 100),
                     layer("mlstm", mlstm(2, 24, 16, cap=4.0), None)]}

TINY_Q = {"architecture": ARCH, "vocab": 97, "width": 40, "norm": {"eps": 1e-6}, "embedding": {"scale": 1.0},
          "canon": {"taps": 1},
          "layers": [layer("mlstm", mlstm(1, 16, 40), 56),
                     layer("attention", attention(2, 2, 32, 24, window=8, conv=0, coef=0.9, every=1, softcap=20.0), 56),
                     layer("attention", attention(4, 1, 16, 16, window=1, conv=5, scale=1.0), 64)]}

TINY_R = {"architecture": ARCH, "vocab": 300, "width": 96, "norm": {"eps": 1e-5}, "embedding": {"scale": 9.0},
          "canon": {"taps": 4},
          "layers": [layer("attention", attention(4, 2, 80, 96, window=40, conv=4, scale=0.11, every=16), 160),
                     layer("mlstm", mlstm(2, 80, 96), 160),
                     layer("attention", attention(4, 2, 80, 96, window=33, conv=2, scale=0.2, kv_from=0), 128)]}

TINY_S = {"architecture": ARCH, "vocab": 120, "width": 48, "norm": {"eps": 1e-5}, "embedding": {"scale": 2.0},
          "canon": {"taps": 2},
          "layers": [layer("mlstm", mlstm(2, 20, 36), 64), layer("mlstm", mlstm(4, 8, 12, cap=5.0), None)]}

TINY_T = {"architecture": ARCH, "vocab": 150, "width": 60, "norm": {"eps": 1e-5}, "embedding": {"scale": 3.0},
          "canon": {"taps": 5},
          "layers": [layer("attention", attention(5, 1, 24, 48, window=19, conv=3), None),
                     layer("attention", attention(5, 1, 24, 48, window=50, conv=4, softcap=0.0, coef=0.0, kv_from=0), None)]}

# name -> (config, page size, weight std, norm std, seed)
TINY = {"P": (TINY_P, 4, 0.15, 0.1, 5), "Q": (TINY_Q, 8, 0.2, 0.2, 6), "R": (TINY_R, 16, 0.1, 0.1, 7),
        "S": (TINY_S, 16, 0.2, 0.1, 8), "T": (TINY_T, 16, 0.2, 0.1, 9)}


def make_model_dir(tmp_path, name: str) -> str:
    raw, _, std, norm_std, seed = TINY[name]
    d = os.path.join(str(tmp_path), f"gufasun_{name}")
    write_random_model(d, ARCH, GufasunConfig.from_dict(raw), seed=seed, std=std, norm_std=norm_std)
    # Gates as a trained model has them: input gates that differ by a few times, not by thousands (else one token
    # owns the memory and the output's sign hangs on the last bits of one dot product), and forget gates near one, so
    # that what an early token left still counts a hundred tokens later.
    path = os.path.join(d, "model.safetensors")
    tensors = load_file(path)
    for name, t in tensors.items():
        if name.endswith((".mix.i", ".mix.f")):
            tensors[name] = (t.float() * 0.2).to(t.dtype)
        elif name.endswith(".mix.f.b"):
            tensors[name] = (t.float() + 4.0).to(t.dtype)
    save_file(tensors, path)
    return d
