"""A selective state-space mixer ("Mamba"): a gated recurrence per channel whose step size, input and output
maps depend on the token.

With ``inner`` channels, ``state`` states per channel, a step-size rank ``dt_rank`` and a short convolution of ``conv``
taps, for a request's tokens t = 0, 1, ...:

    [x | z] = W_in h                                   (inner each)
    u_t = silu(conv_b + sum_j conv[:, j] x_{t - (conv - 1) + j})     per channel; the last column is the current token's,
                                                                     inputs before the request's start are zero
    [d | B | C] = W_x u_t                              (dt_rank, state, state)
    dt = softplus(W_dt d + dt_b)                       per channel
    S_t[c, n] = exp(dt_c A[c, n]) S_{t-1}[c, n] + dt_c u_c B_n,   A = -exp(A_log),  S_{-1} = 0
    y_c = sum_n S_t[c, n] C_n + D_c u_c
    out = W_o (y * silu(z))

What a request carries from step to step is its S (float32) and the convolution's last conv - 1 inputs: one row of
the engine's per-request state (``StateSpec``), laid out as the kernels of ``csrc/ssm.hip`` want it, zeroed when the
request starts.  Nothing is kept per token, so the layer owns no cache pages.  Step sizes, decays, the recurrence and
its sums are float whatever the activation type; the projections and the convolution follow the activation type.

Tensors (``tensors`` maps the roles "in", "conv", "conv_bias", "x", "dt", "dt_bias", "A_log", "D", "out" to full names;
by default ``<name>.in_proj.weight``, ``<name>.conv1d.weight`` [inner, conv], ``<name>.conv1d.bias``,
``<name>.x_proj.weight``, ``<name>.dt_proj.weight``, ``<name>.dt_proj.bias``, ``<name>.A_log``, ``<name>.D``,
``<name>.out_proj.weight``).  W_x is cut at load into the step-size rows and the B/C rows: two products, whose outputs
the next kernels read as they are.
"""
from __future__ import annotations

from typing import Dict, Mapping, Optional

import torch

from ..kernels import ops
from .base import Mixer, MixerBinding, register_part
from .plan import ParamSpec, StateSpec


SCAN_CHUNK = 64             # rows of a chunk of the scan where long portions are cut into chunks that run side by side
SCAN_CHUNK_MIN_ROWS = 128   # ... which happens in steps that bring some request this many rows or more


@register_part("mixer", "selective_ssm")
class SelectiveSSM(Mixer):
    graph_safe = True          # every kernel reads the step's layout from the context's device arrays
    adds_to_stream = True

    def __init__(self, name: str, hidden_size: int, inner: int, state: int, dt_rank: int, conv: int,
                 init_std: float = 0.02, tensors: Optional[Mapping[str, str]] = None):
        self.name, self.hidden_size = name, int(hidden_size)
        self.inner, self.n_state, self.dt_rank, self.taps = int(inner), int(state), int(dt_rank), int(conv)
        if min(self.inner, self.n_state, self.dt_rank, self.taps) <= 0:
            raise ValueError(f"{name}: inner, state, dt_rank and conv must be positive")
        if self.taps > 16 or self.n_state > 128:
            raise ValueError(f"{name}: at most 16 taps and 128 states per channel (got {self.taps}, {self.n_state})")
        self.init_std = init_std
        self.names = {"in": f"{name}.in_proj.weight", "conv": f"{name}.conv1d.weight", "conv_bias": f"{name}.conv1d.bias",
                      "x": f"{name}.x_proj.weight", "dt": f"{name}.dt_proj.weight", "dt_bias": f"{name}.dt_proj.bias",
                      "A_log": f"{name}.A_log", "D": f"{name}.D", "out": f"{name}.out_proj.weight"}
        self.names.update(tensors or {})
        self.conv_floats = self.inner * (self.taps - 1)          # the convolution's part of a state row comes first
        self.w_in = self.w_x_dt = self.w_x_bc = self.w_dt = self.w_o = None
        self.conv_w = self.conv_b = self.dt_b = self.A = self.D = None

    def state_spec(self) -> StateSpec:
        return StateSpec((self.conv_floats + self.inner * self.n_state,), "float32")

    def param_specs(self) -> Dict[str, ParamSpec]:
        nm, H, C, N, R, s = self.names, self.hidden_size, self.inner, self.n_state, self.dt_rank, ("normal", self.init_std)
        return {
            nm["in"]: ParamSpec((2 * C, H), s), nm["conv"]: ParamSpec((C, self.taps), ("normal", 0.3)),
            nm["conv_bias"]: ParamSpec((C,), s), nm["x"]: ParamSpec((R + 2 * N, C), ("normal", 0.1)),
            nm["dt"]: ParamSpec((C, R), ("normal", 0.1)), nm["dt_bias"]: ParamSpec((C,), ("uniform", -4.0, -1.0)),
            nm["A_log"]: ParamSpec((C, N), ("log_uniform", 1.0, 16.0)), nm["D"]: ParamSpec((C,), ("ones",)),
            nm["out"]: ParamSpec((H, C), s),
        }

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        nm, R = self.names, self.dt_rank
        self.w_in = ops.prepare_linear(tensors[nm["in"]])
        w_x = tensors[nm["x"]]
        self.w_x_dt = ops.prepare_linear(w_x[:R].contiguous())
        self.w_x_bc = ops.prepare_linear(w_x[R:].contiguous())
        self.w_dt = ops.prepare_linear(tensors[nm["dt"]])
        self.w_o = ops.prepare_linear(tensors[nm["out"]])
        self.conv_w, self.conv_b = tensors[nm["conv"]].contiguous(), tensors[nm["conv_bias"]]
        if self.conv_b.dtype != self.conv_w.dtype:
            self.conv_w, self.conv_b = self.conv_w.float(), self.conv_b.float()
        self.dt_b, self.D = tensors[nm["dt_bias"]], tensors[nm["D"]]
        if self.dt_b.dtype != self.D.dtype:
            self.dt_b, self.D = self.dt_b.float(), self.D.float()
        self.A = (-torch.exp(tensors[nm["A_log"]].float())).contiguous()        # float whatever the file holds

    def accepts_scaled_rows(self, n_rows: int) -> bool:
        return ops.takes_scaled_rows(n_rows, self.w_in)

    def forward(self, h, ctx, binding: MixerBinding, sink=None):
        state, C, t = binding.state, self.inner, ctx.timer
        if state is None:
            raise ValueError(f"{self.name}: the mixer was given no per-request state")
        xz = ops.linear(h, self.w_in)                                   # [T, 2 inner]: x | z
        u = ops.causal_conv_silu(xz, C, self.conv_w, self.conv_b, state, ctx.row_req, ctx.q_start, ctx.q_len, ctx.state_slots)
        if t is not None:
            t.mark("mixer.conv")
        d = ops.linear(u, self.w_x_dt)                                  # [T, dt_rank]
        bc = ops.linear(u, self.w_x_bc)                                 # [T, 2 state]: B | C
        dt_raw = ops.linear(d, self.w_dt, out_dtype=torch.float32)      # [T, inner] float: the step sizes are never rounded
        # A prompt's portion walked token by token leaves most of the chip idle (the recurrence of a channel is a chain):
        # in bfloat16 long portions are cut into chunks that run side by side.  In 32-bit the walk stays in one piece, so
        # that a token's sums do not depend on where its request was cut.  (Steps of single tokens, the ones that are
        # captured and replayed, never take the chunks: a layout's launches stay the same.)
        chunks = None
        if u.dtype == torch.bfloat16 and ctx.n_tokens > ctx.n_requests and int(ctx.h_q_len.max()) >= SCAN_CHUNK_MIN_ROWS:
            chunks = ctx.derived(("scan_chunks", SCAN_CHUNK), lambda: ops.scan_chunks(ctx.h_q_start, ctx.h_q_len, SCAN_CHUNK, ctx.device))
        y = ops.selective_scan(u, dt_raw, self.dt_b, self.A, bc, self.D, xz[:, C:], state, self.conv_floats,
                               ctx.q_start, ctx.q_len, ctx.state_slots, chunks)
        if t is not None:
            t.mark("mixer.scan")
        if sink is not None and ops.adds_into_stream(y.shape[0], self.w_o, sink.norm_weight):
            return ops.linear_into_stream(y, self.w_o, sink.stream, sink.norm_weight, sink.eps, sink.mult)
        return ops.linear(y, self.w_o, keep_slices=sink is not None)
