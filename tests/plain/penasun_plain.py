"""A plain, slow Penasun in float64 torch on the CPU, one function per mechanism, written from
the design's equations and sharing nothing with the library. It reads config.json with `json`
and model.safetensors with the safetensors package.

Notation: x the residual stream [T, D]; p the position of a token in its sequence (from 0).
State-space mixer: R heads of width P, state size N, Q groups of B/C vectors, K convolution
taps. Attention: H query heads, G key/value heads, key width d, value width e, two score maps
a head. Router: E experts of which the last I have no weights, k chosen a token.
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


# ---- small functions -------------------------------------------------------------

def rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.logaddexp(z, torch.zeros_like(z))


# ---- state-space mixer -----------------------------------------------------------

def causal_conv(u, taps, bias, history=None):
    """u [T, C], taps [C, K] (the last column weighs the present token), history [K-1, C] the
    inputs before u (zeros at a sequence's start). Returns (silu(conv) [T, C], new history)."""
    T, C = u.shape
    K = taps.shape[1]
    if history is None:
        history = torch.zeros((K - 1, C), dtype=u.dtype)
    ext = torch.cat([history, u], 0)                    # ext[t + K - 1] is u[t]
    out = torch.zeros((T, C), dtype=u.dtype)
    for t in range(T):
        for j in range(K):
            out[t] += taps[:, j] * ext[t + j]
    return silu(out + bias), ext[ext.shape[0] - (K - 1):].clone()


def selective_scan(xs, Bs, Cs, dt, A_log, D, state=None):
    """xs [T, R, P], Bs and Cs [T, Q, N], dt [T, R] (already positive), state [R, N, P].
    S <- exp(-exp(A_log_r) dt) S + dt B x^T;  y = S^T C + D_r x. Returns (y [T, R, P], state)."""
    T, R, P = xs.shape
    Q, N = Bs.shape[1], Bs.shape[2]
    if state is None:
        state = torch.zeros((R, N, P), dtype=xs.dtype)
    state = state.clone()
    y = torch.zeros_like(xs)
    for t in range(T):
        for r in range(R):
            q = r // (R // Q)
            decay = math.exp(-math.exp(float(A_log[r])) * float(dt[t, r]))
            state[r] = decay * state[r] + float(dt[t, r]) * torch.outer(Bs[t, q], xs[t, r])
            y[t, r] = state[r].T @ Cs[t, q] + D[r] * xs[t, r]
    return y, state


def gated_group_norm(y, z, weight, parts, eps):
    """y, z [T, W]: y * silu(z), cut into `parts` equal stretches, each divided by its own root
    mean square, times weight."""
    T, W = y.shape
    g = (y * silu(z)).reshape(T, parts, W // parts)
    return rms(g, eps).reshape(T, W) * weight


def mamba2_mixer(h, w, pre, m, eps, carry=None):
    """h [T, D] -> [T, D]; carry = (conv history, state) of the sequence or None at its start."""
    R, P, N, Q = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = R * P
    proj = h @ w[pre + "in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * Q * N], proj[:, 2 * inner + 2 * Q * N:]
    hist, state = carry if carry is not None else (None, None)
    xbc, hist = causal_conv(xbc, w[pre + "conv"], w[pre + "conv.b"], hist)
    T = h.shape[0]
    xs = xbc[:, :inner].reshape(T, R, P)
    Bs = xbc[:, inner:inner + Q * N].reshape(T, Q, N)
    Cs = xbc[:, inner + Q * N:].reshape(T, Q, N)
    dt = softplus(dt + w[pre + "dt_bias"])
    y, state = selective_scan(xs, Bs, Cs, dt, w[pre + "A_log"], w[pre + "D"], state)
    out = gated_group_norm(y.reshape(T, inner), z, w[pre + "norm"], m["norm_groups"], eps)
    return out @ w[pre + "o"].T, (hist, state)


# ---- differential attention --------------------------------------------------------

def query_temperature(p: int, coef: float, every: int) -> float:
    return 1.0 + coef * math.log((p + 1) // every + 1)


def softmax_attention(q, k, v, scale, first_pos):
    """q [T, d] at positions first_pos.., k [S, d], v [S, e] at positions 0..: causal."""
    T = q.shape[0]
    out = torch.zeros((T, v.shape[1]), dtype=q.dtype)
    for t in range(T):
        n = first_pos + t + 1
        s = (k[:n] @ q[t]) * scale
        out[t] = torch.softmax(s, 0) @ v[:n]
    return out


def difference_lambda(w, pre, diff):
    return math.exp(float((w[pre + "lq1"] * w[pre + "lk1"]).sum())) \
        - math.exp(float((w[pre + "lq2"] * w[pre + "lk2"]).sum())) + diff


def diff_attention(h, w, pre, m, eps, carry=None):
    """h [T, D] -> [T, D]; carry = (k [S, G, 2, d], v [S, G, e]) of the tokens before."""
    H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = (h @ w[pre + "q"].T + w[pre + "q.b"]).reshape(T, H, 2, d)
    k = (h @ w[pre + "k"].T + w[pre + "k.b"]).reshape(T, G, 2, d)
    v = (h @ w[pre + "v"].T + w[pre + "v.b"]).reshape(T, G, e)
    first = 0
    if carry is not None:
        first = carry[0].shape[0]
        k = torch.cat([carry[0], k], 0)
        v = torch.cat([carry[1], v], 0)
    qt = m.get("q_temp")
    if qt:
        for t in range(T):
            q[t] = q[t] * query_temperature(first + t, qt["coef"], qt["every"])
    lam = difference_lambda(w, pre, m["diff"])
    heads = []
    for hh in range(H):
        g = hh // (H // G)
        a1 = softmax_attention(q[:, hh, 0], k[:, g, 0], v[:, g], m["scale"], first)
        a2 = softmax_attention(q[:, hh, 1], k[:, g, 1], v[:, g], m["scale"], first)
        heads.append(rms(a1 - lam * a2, eps) * (1.0 - m["diff"]))
    o = torch.cat(heads, 1)
    return o @ w[pre + "o"].T + w[pre + "o.b"], (k, v)


# ---- routed feed-forward -----------------------------------------------------------

def bounded_expert(h, gate, up, down, limit):
    g = torch.clamp(h @ gate.T, max=limit)
    u = torch.clamp(h @ up.T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ down.T


def route(logits, correction, r):
    """logits [E] of one token -> [(expert, weight)], k entries. Scores are a softmax over all E;
    the choice is made on score + correction among the experts of the `keep` groups whose best
    such number is largest; the weight is the plain score times r.scale."""
    E = logits.shape[0]
    s = torch.softmax(logits, 0)
    c = s + correction
    groups = r.get("groups") or {"count": 1, "keep": 1}
    n, keep = groups["count"], groups["keep"]
    size = E // n
    best = torch.stack([c[g * size:(g + 1) * size].max() for g in range(n)])
    kept = torch.topk(best, keep).indices.tolist()
    masked = torch.full_like(c, -math.inf)
    for g in kept:
        masked[g * size:(g + 1) * size] = c[g * size:(g + 1) * size]
    chosen = torch.topk(masked, r["top"]).indices.tolist()
    return [(e, float(s[e]) * r["scale"]) for e in chosen]


def routed_ff(h, w, pre, mlp):
    r = mlp["router"]
    real = r["experts"]                      # the router has real + identity outputs
    out = torch.zeros_like(h)
    logits = h @ w[pre + "router"].T
    for t in range(h.shape[0]):
        for e, weight in route(logits[t], w[pre + "correction"], r):
            if e >= real:
                out[t] += weight * h[t]
            else:
                out[t] += weight * bounded_expert(h[t], w[f"{pre}e{e}.gate"], w[f"{pre}e{e}.up"],
                                                  w[f"{pre}e{e}.down"], mlp["expert"]["limit"])
    return out


# ---- the model ---------------------------------------------------------------------

def forward(cfg, w, tokens, carry=None, layers_out=None):
    """Logits [T, vocab] of `tokens` that continue the sequence `carry` describes (None: its
    start). Returns (logits, carry). layers_out: a list that receives x after every layer."""
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.tensor(tokens)]
    carry = list(carry) if carry is not None else [None] * len(cfg["layers"])
    for i, layer in enumerate(cfg["layers"]):
        pre = f"l{i}."
        n = rms(x, eps) * w[pre + "norm1"]
        if layer["type"] == "mamba2":
            d, carry[i] = mamba2_mixer(n, w, pre + "mix.", layer["mixer"], eps, carry[i])
        elif layer["type"] == "attention":
            d, carry[i] = diff_attention(n, w, pre + "mix.", layer["mixer"], eps, carry[i])
        else:
            raise ValueError(layer["type"])
        x = x + d
        if layer.get("mlp") is not None:
            x = x + routed_ff(rms(x, eps) * w[pre + "norm2"], w, pre + "mlp.", layer["mlp"])
        if layers_out is not None:
            layers_out.append(x.clone())
    return (rms(x, eps) * w["final.norm"]) @ w["embed"].T, carry


def greedy(cfg, w, prompt, steps: int) -> list[int]:
    """`steps` tokens after `prompt`, each the argmax of the last logits (lowest id on ties)."""
    logits, carry = forward(cfg, w, list(prompt))
    out = []
    for _ in range(steps):
        t = int(torch.argmax(logits[-1]))
        out.append(t)
        logits, carry = forward(cfg, w, [t], carry)
    return out
