"""Volonex as data: a decoder whose layers each name their own sizes.

Token embedding times a constant; per layer a pre-norm block with a residual multiplier m,
x += m * attention(norm1(x)) and, where the layer has one, x += m * ff(norm2(x)); the norms
are Dynamic Tanh (tanh(alpha x) * w + b); attention is grouped-query with separate key and
value widths, an interleaved partial rotation with YaRN-scaled frequencies, a score scale of
its own, a chunked causal mask, a per-head sink in the softmax and a per-head sigmoid gate on
the output; the feed-forward is gated with a bounded gate and up, g' * sigmoid(1.702 g') *
(u' + 1). A stretch of layers may run several times in a row with the same weights, each pass
with a cache of its own, the embedding's output added again before every pass but the first.
Final Dynamic Tanh, then an output matrix of its own.

Tensor names: 'embed', 'head', 'final.norm' (+ '.b', '.alpha'), and per layer i 'l<i>.norm1',
'l<i>.norm2' (+ '.b', '.alpha'), 'l<i>.mix.{q,k,v,o,g,sink}', 'l<i>.mlp.{gate,up,down}'.
"""
from __future__ import annotations

from ..config.volonex import VolonexConfig
from ..parts.base import LayerSpec, ModelSpec, PartSpec, ScheduleEntry
from ..registry import register_architecture

# positions are exact in the fp32 angles up to 2^24; the configuration names no bound of its own
_MAX_POSITIONS = 1 << 22


def volonex_spec(cfg: VolonexConfig) -> ModelSpec:
    norm = PartSpec("dynamic_tanh", {"size": cfg.width, "names": {"weight": "", "bias": "b", "alpha": "alpha"}})
    layers = []
    for l, layer in enumerate(cfg.layers):
        a = layer.mixer
        position = PartSpec("none")
        if a.rot is not None:
            params = {"head_dim": a.dim, "rotary_dim": a.rot.dims, "theta": a.rot.base, "interleaved": True}
            if a.rot.scaling is not None:
                params["scaling"] = {"kind": "yarn", **a.rot.scaling.to_dict()}
            position = PartSpec("rotary", params)
        mixer = PartSpec("attention", {
            "hidden_size": cfg.width, "num_heads": a.heads, "num_kv_heads": a.kv_heads,
            "head_dim": a.dim, "value_dim": a.vdim, "scale": a.scale, "chunk": a.chunk,
            "sinks": True, "head_gate": True, "qkv_bias": False, "out_bias": False,
            "position": position,
            "names": {"q": "q", "k": "k", "v": "v", "o": "o", "gate": "g", "sinks": "sink"},
        })
        params = {"mixer_norm": norm, "mixer": mixer, "residual_scale": cfg.residual_mult,
                  "names": {"mixer_norm": "norm1", "mixer": "mix",
                            "feed_forward_norm": "norm2", "feed_forward": "mlp"}}
        if layer.mlp is not None:
            params["feed_forward_norm"] = norm
            params["feed_forward"] = PartSpec("gated_mlp", {
                "hidden_size": cfg.width, "intermediate_size": layer.mlp.ff,
                "activation": "clamped_swiglu", "limit": layer.mlp.limit, "alpha": 1.702,
                "names": {"gate": "gate", "up": "up", "down": "down"}})
        layers.append(LayerSpec(f"l{l}.", PartSpec("pre_norm", params)))
    return ModelSpec(
        hidden_size=cfg.width,
        vocab_size=cfg.vocab,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab, "hidden_size": cfg.width,
                                               "scale": cfg.embedding_scale, "names": {"weight": ""}}),
        embedding_prefix="embed.",
        layers=layers,
        schedule=[ScheduleEntry(l, add_embedding=again) for l, again in cfg.runs()],
        final_norm=norm,
        final_norm_prefix="final.norm.",
        head=PartSpec("linear_head", {"vocab_size": cfg.vocab, "hidden_size": cfg.width, "names": {"weight": ""}}),
        head_prefix="head.",
        max_positions=_MAX_POSITIONS,
    )


register_architecture("Volonex", VolonexConfig, volonex_spec)
