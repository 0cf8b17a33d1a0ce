"""A plain, slow Volonex in float64 torch on the CPU, one function per mechanism, written from
the design's equations and sharing nothing with the library. It reads config.json with `json`
and model.safetensors with the safetensors package.

Notation: x the residual stream [T, D]; p the position of a token in its sequence (from 0);
m the residual multiplier; H query heads, G key/value heads, d the query/key width, e the value
width of a head.
"""
from __future__ import annotations

import json
import math
import os

import torch

F64 = torch.float64


def read_model(folder: str):
    """(config dict, {name: float64 tensor})."""
    from safetensors.torch import load_file
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    w = {k: (v.to(F64) if v.is_floating_point() else v) for k, v in
         load_file(os.path.join(folder, "model.safetensors")).items()}
    return cfg, w


# ---- mechanisms ----------------------------------------------------------------

def dynamic_tanh(x, weight, bias, alpha):
    """y = tanh(alpha x) * weight + bias: no mean, no variance."""
    return torch.tanh(alpha * x) * weight + bias


def rotary_frequencies(rot: dict):
    """(f [dims/2], multiplier of cos and sin). f_i = base^(-2i/dims); with 'scaling' the slow
    frequencies are divided by `factor` along a ramp between the dims whose wavelength fits
    `fast` and `slow` times into `original` positions, and cos/sin grow by 0.1 ln(factor) + 1."""
    dims, base = rot["dims"], rot["base"]
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F64)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0

    def dim_of(turns):
        return dims * math.log(sc["original"] / (2 * math.pi * turns)) / (2 * math.log(base))

    lo = max(math.floor(dim_of(sc["fast"])), 0)
    hi = min(math.ceil(dim_of(sc["slow"])), dims - 1)
    out = f.clone()
    for i in range(dims // 2):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out[i] = f[i] / sc["factor"] * ramp + f[i] * (1 - ramp)
    return out, 0.1 * math.log(sc["factor"]) + 1.0


def rotate_interleaved(x, positions, rot: dict | None, single: bool = False):
    """x [T, heads, d]: dims (2i, 2i+1) of the first rot.dims turn by the angle p f_i, the rest
    pass: (u, v) -> (u cos - v sin, v cos + u sin), cos and sin times the multiplier. single: the
    frequency and the angle are rounded to 32-bit floats, as the design computes them (at
    positions in the thousands that rounding is what decides the last digits)."""
    if not rot:
        return x
    f, mult = rotary_frequencies(rot)
    y = x.clone()
    for t, p in enumerate(positions):
        for i in range(rot["dims"] // 2):
            a = float(p) * float(f[i])
            if single:
                a = float(torch.tensor(float(p), dtype=torch.float32) * f[i].to(torch.float32))
            c, s = math.cos(a) * mult, math.sin(a) * mult
            u, v = x[t, :, 2 * i], x[t, :, 2 * i + 1]
            y[t, :, 2 * i] = u * c - v * s
            y[t, :, 2 * i + 1] = v * c + u * s
    return y


def sees(i: int, j: int, chunk: int, window: int = 0) -> bool:
    """Whether position i attends position j."""
    if j > i:
        return False
    if chunk and i // chunk != j // chunk:
        return False
    if window and j <= i - window:
        return False
    return True


def softmax_with_sink(scores, sink):
    """Weights of the keys when the denominator also holds exp(sink) (one more term that has no
    value): a vector that sums to less than 1."""
    m = max(float(scores.max()), float(sink))
    e = torch.exp(scores - m)
    return e / (e.sum() + math.exp(float(sink) - m))


def attention(h, positions, mx: dict, w: dict, prefix: str, k_cache=None, v_cache=None, past=()):
    """h [T, D] the mixer's input at `positions`; `past` are earlier positions whose rotated keys
    and values are in k_cache / v_cache (lists, appended to here). Returns [T, D]."""
    H, G, d, e = mx["heads"], mx.get("kv_heads", mx["heads"]), mx["dim"], mx.get("vdim", mx["dim"])
    T = h.shape[0]
    q = (h @ w[prefix + "q"].T).view(T, H, d)
    k = (h @ w[prefix + "k"].T).view(T, G, d)
    v = (h @ w[prefix + "v"].T).view(T, G, e)
    q = rotate_interleaved(q, positions, mx.get("rot"))
    k = rotate_interleaved(k, positions, mx.get("rot"))
    gate = torch.sigmoid(h @ w[prefix + "g"].T)            # [T, H]
    keys = list(k_cache or []) + [k[t] for t in range(T)]
    vals = list(v_cache or []) + [v[t] for t in range(T)]
    where = list(past) + list(positions)
    if k_cache is not None:
        k_cache[:] = keys
        v_cache[:] = vals
    chunk = (mx.get("mask") or {}).get("size", 0)
    out = torch.zeros(T, H, e, dtype=F64)
    all_k, all_v = torch.stack(keys), torch.stack(vals)        # [n, G, d], [n, G, e]
    for t, p in enumerate(positions):
        js = [n for n, pj in enumerate(where) if sees(p, pj, chunk)]
        for head in range(H):
            kv = head // (H // G)
            s = (all_k[js, kv] @ q[t, head]) * mx["scale"]       # one score a visible key
            a = softmax_with_sink(s, w[prefix + "sink"][head])
            out[t, head] = (a @ all_v[js, kv]) * gate[t, head]
    return out.reshape(T, H * e) @ w[prefix + "o"].T


def bounded_gated(h, mlp: dict, w: dict, prefix: str):
    lim = mlp["limit"]
    g = torch.clamp(h @ w[prefix + "gate"].T, max=lim)
    u = torch.clamp(h @ w[prefix + "up"].T, -lim, lim)
    return (g * torch.sigmoid(1.702 * g) * (u + 1)) @ w[prefix + "down"].T


def runs(cfg: dict):
    """[(layer, whether the embedding is added before it)] in running order."""
    n = len(cfg["layers"])
    lp = cfg.get("loop") or {"start": 0, "stop": 0, "times": 1}
    order = [(l, False) for l in range(lp["start"])]
    for t in range(lp["times"]):
        order += [(l, t > 0 and l == lp["start"]) for l in range(lp["start"], lp["stop"])]
    return order + [(l, False) for l in range(lp["stop"], n)]


def norm(x, w, name):
    return dynamic_tanh(x, w[name], w[name + ".b"], w[name + ".alpha"])


def embed(cfg, w, ids):
    return w["embed"][torch.tensor(list(ids), dtype=torch.long)] * (cfg.get("embedding") or {}).get("scale", 1.0)


class State:
    """The keys and values of every run of one sequence, and its length."""

    def __init__(self, cfg):
        self.k = [[] for _ in runs(cfg)]
        self.v = [[] for _ in runs(cfg)]
        self.length = 0


def step(cfg, w, state: State, ids):
    """Feeds ids behind what the state holds; logits [len(ids), vocab] in float64."""
    positions = list(range(state.length, state.length + len(ids)))
    past = list(range(state.length))
    x = embed(cfg, w, ids)
    x0 = x.clone()
    m = cfg.get("residual_mult", 1.0)
    for r, (l, again) in enumerate(runs(cfg)):
        layer = cfg["layers"][l]
        if again:
            x = x + x0
        x = x + m * attention(norm(x, w, f"l{l}.norm1"), positions, layer["mixer"], w, f"l{l}.mix.",
                              state.k[r], state.v[r], past)
        if layer.get("mlp"):
            x = x + m * bounded_gated(norm(x, w, f"l{l}.norm2"), layer["mlp"], w, f"l{l}.mlp.")
    state.length += len(ids)
    return norm(x, w, "final.norm") @ w["head"].T


def forward(cfg, w, ids):
    return step(cfg, w, State(cfg), ids)


def greedy(cfg, w, prompt, n_new):
    st = State(cfg)
    logits = step(cfg, w, st, prompt)
    out = []
    for _ in range(n_new):
        out.append(int(logits[-1].argmax()))
        logits = step(cfg, w, st, [out[-1]])
    return out
