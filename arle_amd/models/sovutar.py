"""Recipe of the Sovutar decoder: its configuration written out as a ModelSpec.

Every layer is a `post_norm` block: the mixer and the feed-forward read the residual itself, and an RMS norm whose
weight is stored around zero stands on each one's output before it is added.  The mixer is a chunked attention whose q
and k are normed over the whole projection and whose values are mixed with those of the first such layer
(`wide_norm_attention`), or a latent attention over a sliding window with a sink in the softmax (`latent_attention`,
rotation `rope_interleaved`).  The feed-forward is a mixture of experts with a sigmoid router and a shared expert
(`sigmoid_moe`).  The final norm is of the same one-plus kind; the head caps its logits.  Tensor names: `embed`,
`l<i>.norm1|norm2`, `l<i>.mix.*`, `l<i>.mlp.*`, `final.norm`, `head`.
"""
from __future__ import annotations

from ..config.registry import register_architecture
from ..config.sovutar import ARCHITECTURE, ChunkedAttentionConfig, SovutarConfig
from ..parts.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

# the rotation's table is made for the longest request the engine is built for, not for a number of the model's
MAX_POSITIONS = 1 << 30


def _chunked(c: SovutarConfig, i: int, p: str) -> PartSpec:
    m = c.layers[i].mixer
    first = c.first_value_mixer()
    role = None if not m.v_mix else ("source" if i == first else "mix")
    params = {"hidden_size": c.width, "num_q_heads": m.heads, "num_kv_heads": m.kv_heads, "key_dim": m.dim,
              "value_dim": m.vdim, "qk_norm": True, "eps": c.eps, "scale": m.scale, "chunk": m.chunk, "window": None,
              "value_mix": role, "carry_key": "first_values"}
    weights = {"q": p + "q", "k": p + "k", "v": p + "v", "o": p + "o", "q_norm": p + "q.norm", "k_norm": p + "k.norm"}
    if role == "mix":
        weights["mix"] = p + "vmix"
    return PartSpec("wide_norm_attention", params, weights)


def _latent(c: SovutarConfig, i: int, p: str) -> PartSpec:
    m = c.layers[i].mixer
    position = PartSpec("rope_interleaved", {"head_dim": m.rot_dim, "rotary_dim": m.rot_dims, "theta": m.rot_base,
                                             "max_positions": 1})
    params = {"hidden_size": c.width, "heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "value_dim": m.vdim,
              "rank": m.kv_rank, "eps": c.eps, "scale": m.scale, "window": m.window, "sink": True, "position": position}
    return PartSpec("latent_attention", params,
                    {"q": p + "q", "dkv": p + "dkv", "c_norm": p + "dkv.norm", "uk": p + "uk", "uv": p + "uv",
                     "sink": p + "sink", "o": p + "o"})


def _moe(c: SovutarConfig, i: int, p: str) -> PartSpec:
    m = c.layers[i].mlp
    params = {"hidden_size": c.width, "experts": m.experts, "top": m.top, "expert_size": m.expert_ff, "scale": m.scale,
              "correction": True, "shared_size": m.shared_ff,
              "shared_weights": {"gate": p + "shared.gate", "up": p + "shared.up", "down": p + "shared.down"}}
    weights = {"router": p + "router", "correction": p + "correction"}
    for e in range(m.experts):
        weights.update({f"gate{e}": f"{p}e{e}.gate", f"up{e}": f"{p}e{e}.up", f"down{e}": f"{p}e{e}.down"})
    return PartSpec("sigmoid_moe", params, weights)


def sovutar_spec(config: SovutarConfig, stop_token_ids=()) -> ModelSpec:
    c = config
    norm = lambda tensor: PartSpec("rmsnorm", {"width": c.width, "eps": c.eps, "one_plus": True}, {"weight": tensor})
    layers, schedule = [], []
    for i, layer in enumerate(c.layers):
        p = f"l{i}."
        build = _chunked if isinstance(layer.mixer, ChunkedAttentionConfig) else _latent
        norms = {"mixer_out": norm(p + "norm1")}
        ffn = None
        if layer.mlp is not None:
            norms["ffn_out"] = norm(p + "norm2")
            ffn = _moe(c, i, p + "mlp.")
        layers.append(LayerSpec("post_norm", build(c, i, p + "mix."), ffn, norms))
        schedule.append(ScheduleEntry(i))
    sizes = {"vocab_size": c.vocab, "hidden_size": c.width}
    return ModelSpec(hidden_size=c.width, vocab_size=c.vocab, max_positions=MAX_POSITIONS,
                     embedding=PartSpec("token_table", sizes, {"table": "embed"}),
                     layers=layers, schedule=schedule, final_norm=norm("final.norm"),
                     head=PartSpec("linear", dict(sizes, softcap=c.logit_softcap), {"weight": "head"}),
                     stop_token_ids=tuple(stop_token_ids))


register_architecture(ARCHITECTURE, SovutarConfig, sovutar_spec)
