"""Penasun as data: a decoder whose layers each name their kind and sizes.

Token embedding; per layer a pre-norm block x += mixer(norm1(x)) and, where the layer has one,
x += ff(norm2(x)) with RMS norms; the mixer is either a state-space mixer with a selective scan
(parts/state_space.py) or a differential attention without rotation whose queries get a
temperature that grows with the position (parts/attention.py: score_maps, q_temp); the
feed-forward is routed over experts with bounded gates, identity experts among them, a choice
limited to the best groups of experts and made on corrected scores (parts/routed.py). Final RMS
norm, then the embedding matrix once more as the output matrix.

Tensor names: 'embed', 'final.norm', and per layer i 'l<i>.norm1', 'l<i>.norm2',
'l<i>.mix.{in,conv,conv.b,dt_bias,A_log,D,norm,o}' or 'l<i>.mix.{q,k,v,o}' (+ '.b') with
'l<i>.mix.{lq1,lk1,lq2,lk2}', 'l<i>.mlp.{router,correction}' and 'l<i>.mlp.e<j>.{gate,up,down}'.
"""
from __future__ import annotations

from ..config.penasun import PenasunConfig
from ..parts.base import LayerSpec, ModelSpec, PartSpec, ScheduleEntry
from ..registry import register_architecture

# positions are exact in fp32 up to 2^24; the configuration names no bound of its own
_MAX_POSITIONS = 1 << 22


def penasun_spec(cfg: PenasunConfig) -> ModelSpec:
    norm = PartSpec("rmsnorm", {"size": cfg.width, "eps": cfg.norm_eps, "names": {"weight": ""}})
    layers = []
    for l, layer in enumerate(cfg.layers):
        m = layer.mixer
        if layer.type == "mamba2":
            mixer = PartSpec("mamba2", {
                "hidden_size": cfg.width, "num_heads": m.heads, "head_dim": m.vdim, "state_size": m.state,
                "groups": m.groups, "conv_taps": m.conv, "norm_groups": m.norm_groups, "eps": cfg.norm_eps,
                "names": {"in": "in", "conv": "conv", "conv_bias": "conv.b", "dt_bias": "dt_bias",
                          "A_log": "A_log", "D": "D", "norm": "norm", "o": "o"}})
        else:
            params = {
                "hidden_size": cfg.width, "num_heads": m.heads, "num_kv_heads": m.kv_heads,
                "head_dim": m.dim, "value_dim": m.vdim, "scale": m.scale, "qkv_bias": True, "out_bias": True,
                "score_maps": 2, "diff": m.diff, "diff_eps": cfg.norm_eps, "position": PartSpec("none"),
                "names": {"q": "q", "k": "k", "v": "v", "o": "o", "q_bias": "q.b", "k_bias": "k.b",
                          "v_bias": "v.b", "o_bias": "o.b", "lq1": "lq1", "lk1": "lk1", "lq2": "lq2", "lk2": "lk2"}}
            if m.q_temp_every:
                params["q_temp"] = {"coef": m.q_temp_coef, "every": m.q_temp_every}
            mixer = PartSpec("attention", params)
        params = {"mixer_norm": norm, "mixer": mixer,
                  "names": {"mixer_norm": "norm1", "mixer": "mix", "feed_forward_norm": "norm2", "feed_forward": "mlp"}}
        if layer.mlp is not None:
            f = layer.mlp
            params["feed_forward_norm"] = norm
            params["feed_forward"] = PartSpec("routed_experts", {
                "hidden_size": cfg.width, "intermediate_size": f.ff, "experts": f.experts,
                "identity_experts": f.identity, "top": f.top, "scale": f.scale, "groups": f.group_count,
                "keep_groups": f.group_keep, "correction": True, "limit": f.limit, "alpha": 1.702, "up_shift": 1.0,
                "names": {"router": "router", "correction": "correction", "expert": "e{e}.",
                          "gate": "gate", "up": "up", "down": "down"}})
        layers.append(LayerSpec(f"l{l}.", PartSpec("pre_norm", params)))
    return ModelSpec(
        hidden_size=cfg.width,
        vocab_size=cfg.vocab,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab, "hidden_size": cfg.width,
                                               "names": {"weight": ""}}),
        embedding_prefix="embed.",
        layers=layers,
        schedule=[ScheduleEntry(l) for l in range(len(cfg.layers))],
        final_norm=norm,
        final_norm_prefix="final.norm.",
        head=PartSpec("linear_head", {"vocab_size": cfg.vocab, "hidden_size": cfg.width, "tied_to": "embed"}),
        head_prefix="head.",
        max_positions=_MAX_POSITIONS,
    )


register_architecture("Penasun", PenasunConfig, penasun_spec)
