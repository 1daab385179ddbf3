"""Recipe of the Gufasun decoder: its configuration written out as a ModelSpec.

Every layer is a parallel block: two bias-free layer norms of the same residual feed a mixer and a dense PolyNorm
feed-forward, whose outputs are added to the residual together.  What the mixer reads first passes a short causal
convolution with a residual connection (`input_conv`).  The mixer is a sliding-window, soft-capped attention
without rotation (`softcap_attention`; a layer with `kv_from` reads the pages of an earlier layer, which the
schedule says with `cache_from`) or an mLSTM matrix memory (`mlstm`).  The embedding is scaled, the final norm is
a layer norm, the head is a plain projection.  Tensor names: `embed`, `l<i>.norm1|norm2|canon1`, `l<i>.mix.*`,
`l<i>.mlp.*`, `final.norm`, `head`; a bias is its tensor's name with `.b` added.
"""
from __future__ import annotations

from ..config.gufasun import ARCHITECTURE, AttentionMixer, GufasunConfig
from ..config.registry import register_architecture
from ..parts.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

# the design has no table per position: a request is as long as the cache lets it be
MAX_POSITIONS = 1 << 30


def _attention(c: GufasunConfig, i: int, p: str) -> PartSpec:
    m = c.layers[i].mixer
    shares = m.kv_from is not None
    params = {"hidden_size": c.width, "num_q_heads": m.heads, "num_kv_heads": m.kv_heads, "key_dim": m.dim,
              "value_dim": m.vdim, "bias": True, "conv_taps": m.conv, "qk_norm": True, "eps": c.eps,
              "temp_coef": m.temp_coef, "temp_every": m.temp_every, "scale": m.scale, "softcap": m.softcap,
              "distance_penalty": True, "window": m.window, "cache_window": c.cache_window(i), "shares_kv": shares}
    weights = {"q": p + "q", "q_bias": p + "q.b", "q_norm": p + "q.norm", "r1": p + "r1", "r2": p + "r2", "o": p + "o"}
    if m.conv:
        weights["q_conv"] = p + "q.conv"
    if not shares:
        weights.update({"k": p + "k", "k_bias": p + "k.b", "v": p + "v", "v_bias": p + "v.b", "k_norm": p + "k.norm"})
        if m.conv:
            weights.update({"k_conv": p + "k.conv", "v_conv": p + "v.conv"})
    return PartSpec("softcap_attention", params, weights)


def _mlstm(c: GufasunConfig, i: int, p: str) -> PartSpec:
    m = c.layers[i].mixer
    return PartSpec("mlstm", {"hidden_size": c.width, "heads": m.heads, "key_dim": m.dim, "value_dim": m.vdim,
                              "gate_cap": m.gate_cap, "eps": c.eps},
                    {"q": p + "q", "k": p + "k", "v": p + "v", "g": p + "g", "o": p + "o", "norm": p + "norm",
                     "i": p + "i", "i_bias": p + "i.b", "f": p + "f", "f_bias": p + "f.b"})


def gufasun_spec(config: GufasunConfig, stop_token_ids=()) -> ModelSpec:
    c = config
    norm = lambda tensor: PartSpec("layernorm", {"width": c.width, "eps": c.eps}, {"weight": tensor})
    layers, schedule = [], []
    for i, layer in enumerate(c.layers):
        p = f"l{i}."
        inner = _attention(c, i, p + "mix.") if isinstance(layer.mixer, AttentionMixer) else _mlstm(c, i, p + "mix.")
        mixer = PartSpec("input_conv", {"width": c.width, "taps": c.canon_taps, "inner": inner}, {"weight": p + "canon1"})
        norms = {"mixer_in": norm(p + "norm1")}
        ffn = None
        if layer.ff is not None:
            norms["ffn_in"] = norm(p + "norm2")
            ffn = PartSpec("polynorm", {"hidden_size": c.width, "intermediate_size": layer.ff, "eps": c.eps},
                           {"up": p + "mlp.up", "up_bias": p + "mlp.up.b", "down": p + "mlp.down",
                            "down_bias": p + "mlp.down.b", "coef": p + "mlp.act"})
        layers.append(LayerSpec("parallel", mixer, ffn, norms))
        schedule.append(ScheduleEntry(i, cache_from=getattr(layer.mixer, "kv_from", None)))
    sizes = {"vocab_size": c.vocab, "hidden_size": c.width}
    return ModelSpec(hidden_size=c.width, vocab_size=c.vocab, max_positions=MAX_POSITIONS,
                     embedding=PartSpec("token_table", dict(sizes, scale=c.embedding_scale), {"table": "embed"}),
                     layers=layers, schedule=schedule, final_norm=norm("final.norm"),
                     head=PartSpec("linear", sizes, {"weight": "head"}), stop_token_ids=tuple(stop_token_ids))


register_architecture(ARCHITECTURE, GufasunConfig, gufasun_spec)
