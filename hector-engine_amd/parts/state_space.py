"""A state-space mixer with a selective scan (the "mamba2" kind): no keys and values in the cache,
but a state of fixed size per sequence.

With R heads of P value dims, a state of N dims, Q groups of B / C vectors and K convolution taps
(inner = R P, C = inner + 2 Q N):
    [z | x | B | C | dt] = W_in n                    widths inner, inner, Q N, Q N, R
    [x | B | C] <- silu(causal convolution per channel over the K last inputs + bias)
    dt <- softplus(dt + dt_bias)                     (fp32 from here on)
    per head r, with the B and C of group r // (R / Q):
        S <- exp(-exp(A_log_r) dt_r) S + dt_r B x_r^T,    y_r = S^T C + D_r x_r
    g = y * silu(z), divided by its root mean square in each of `norm_groups` equal stretches, * norm
    out = W_o g
A sequence carries the last K - 1 inputs of the convolution and S (fp32, zeros at its start) in
its row of the cache's state area, which the kernels address on the device through the step's
slots: prompt steps, one-token steps, mixed steps and replayed graphs run the same launches.
names: the suffixes of its tensors (in, conv, conv_bias, dt_bias, A_log, D, norm, o).
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import BuildEnv, LayerCache, Mixer, StepContext, TensorSpec, param, register_part, tensor_name
from .linear import Linear
from ..weights.random_init import register_init

_NAMES = {"in": "in_proj.weight", "conv": "conv1d.weight", "conv_bias": "conv1d.bias", "dt_bias": "dt_bias",
          "A_log": "A_log", "D": "D", "norm": "norm.weight", "o": "out_proj.weight"}

# random values for the tests' and the benchmark's models: decay rates exp(A_log) around 1, step sizes
# softplus(dt + dt_bias) around 0.3, taps that keep the convolution's output of the inputs' size
register_init("ssm_a_log", lambda init: (0.0, 0.5))
register_init("ssm_dt_bias", lambda init: (-1.0, 0.5))


@register_part("mixer", "mamba2")
class SelectiveScanMixer(Mixer):
    accepts_normed_rows = True

    def __init__(self, params: dict, prefix: str, env: BuildEnv):
        super().__init__(prefix, env)
        self.hidden = param(params, "hidden_size", int)
        self.R = param(params, "num_heads", int)
        self.P = param(params, "head_dim", int)
        self.N = param(params, "state_size", int)
        self.Q = param(params, "groups", int, 1)
        self.K = param(params, "conv_taps", int)
        self.parts = param(params, "norm_groups", int, 1)
        self.eps = param(params, "eps", float)
        if min(self.R, self.P, self.N, self.Q, self.K, self.parts) <= 0:
            raise ValueError("mamba2: heads, head_dim, state_size, groups, conv_taps and norm_groups must be positive")
        if self.R % self.Q:
            raise ValueError(f"mamba2: {self.R} heads are not a multiple of {self.Q} groups")
        self.inner = self.R * self.P
        if self.inner % self.parts:
            raise ValueError(f"mamba2: norm_groups {self.parts} does not divide the inner width {self.inner}")
        self.C = self.inner + 2 * self.Q * self.N
        names = param(params, "names", dict, {})
        self._names = {k: tensor_name(prefix, names, k, d) for k, d in _NAMES.items()}
        self.in_proj: Linear | None = None
        self.o_proj: Linear | None = None
        self.taps = self.conv_bias = self.dt_bias = self.a_log = self.d_skip = self.norm = None

    # bytes of the carried convolution inputs, rounded so that the scan's state starts on 16 bytes
    def _conv_bytes(self) -> int:
        return (4 * (self.K - 1) * self.C + 15) // 16 * 16

    def state_bytes(self) -> int:
        return self._conv_bytes() + 4 * self._scan_floats()

    def _scan_floats(self) -> int:
        # the state dims are padded to the scan kernel's share per thread (8 dims, 16 beyond 512, times a
        # power of two of threads), the value dims to its workgroups' (256 threads at most): the same rule
        # as csrc/state_space.hip, kept here so that the cache can be sized where no kernel library is loaded
        npt = 8 if self.N <= 512 else 16
        ng = 1
        while ng * npt < self.N:
            ng *= 2
        pb = min(self.P, 256 // ng)
        return self.R * -(-self.P // pb) * pb * ng * npt

    def tensor_specs(self):
        n = self._names
        return {
            n["in"]: TensorSpec((2 * self.inner + 2 * self.Q * self.N + self.R, self.hidden)),
            n["conv"]: TensorSpec((self.C, self.K), ("normal", 0.3)),
            n["conv_bias"]: TensorSpec((self.C,)),
            n["dt_bias"]: TensorSpec((self.R,), ("ssm_dt_bias",)),
            n["A_log"]: TensorSpec((self.R,), ("ssm_a_log",)),
            n["D"]: TensorSpec((self.R,), ("gain", 1.0, 0.1)),
            n["norm"]: TensorSpec((self.inner,), ("gain", 1.0, 0.1)),
            n["o"]: TensorSpec((self.hidden, self.inner)),
        }

    def bind(self, tensors):
        n = self._names
        self.in_proj = Linear(tensors[n["in"]])
        self.o_proj = Linear(tensors[n["o"]])
        self.taps, self.conv_bias = tensors[n["conv"]].contiguous(), tensors[n["conv_bias"]]
        self.dt_bias, self.a_log, self.d_skip = tensors[n["dt_bias"]], tensors[n["A_log"]], tensors[n["D"]]
        self.norm = tensors[n["norm"]]
        small = (self.taps, self.conv_bias, self.dt_bias, self.a_log, self.d_skip)
        if len({t.dtype for t in small}) != 1:
            raise TypeError(f"{self.prefix}: the convolution's and the scan's parameters are stored in different dtypes")

    def forward(self, x, ctx: StepContext, cache: LayerCache):
        if cache.state is None:
            raise RuntimeError(f"{self.prefix}: a state-space mixer needs its row of the state area")
        rows, inner = ctx.rows, self.inner
        if ops.ssm_state_floats(self.R, self.P, self.N) != self._scan_floats():
            raise RuntimeError(f"{self.prefix}: the scan kernel's state layout differs from the cache's")
        proj = self.in_proj(x, rows, ctx)                       # [rows, z | x B C | dt]
        xbc = ctx.alloc((rows, self.C))
        ops.conv_state(xbc, proj[:, inner:inner + self.C], self.taps, self.conv_bias, cache.state,
                       ctx.positions, ctx.row_seq, ctx.seq_slot, ctx.seq_start, ctx.cu_seqlens,
                       rows, ctx.num_seqs, ctx.all_single)
        y = ctx.alloc((rows, inner), torch.float32)
        if ctx.padded:
            y.zero_()           # the scan writes the rows of sequences only
        ops.ssm_scan(y, xbc, proj[:, inner + self.C:], self.dt_bias, self.a_log, self.d_skip, cache.state,
                     self._conv_bytes(), ctx.cu_seqlens, ctx.seq_slot, rows, ctx.num_seqs,
                     self.R, self.Q, self.N, self.P, max_q_len=ctx.max_q_len)
        g = ctx.alloc((rows, inner))
        ops.gated_group_norm(g, y, proj[:, :inner], self.norm, rows, self.parts, self.eps)
        return self.o_proj(g, rows, ctx, sink=ctx.take_sink())
