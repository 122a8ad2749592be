"""Mixers that keep a matrix of fixed size per request and head instead of keys and values per token.

Both run on one recurrence kernel (`ops.linear_recurrence`): per head a state S [N, P] in float32,
    S_t = a_t * S_(t-1) + b_t * k_t v_t^T,      y_t = S_t^T q_t (+ skip * v_t),
with k_t, q_t of size N (shared by the heads of a group) and v_t of size P. What differs is where a_t and b_t
come from: one fixed decay per head and b = 1 (`LinearAttention`), or a step size per token and head that a
projection gives, a = exp(-rate * dt), b = dt (`SelectiveStateSpace`). The state lives in a request's state
slot; the step function zeroes it when the request's tokens start at position 0, and a step carries it on from
wherever the step before left it, so a prompt may be cut anywhere.
"""
from __future__ import annotations

import math

import torch

from ..kernels import ops
from .base import Mixer, ParamSpec, StateNeed, register_part
from .linear import Linear


@register_part("mixer", "lightning")
class LinearAttention(Mixer):
    """q = silu(W_q x), k = silu(W_k x) ([heads, key_dim]), v = silu(W_v x) ([heads, value_dim]), one packed
    product with a gate of the output's width behind them; S_t = decay_h S_(t-1) + k_t v_t^T, o_t = S_t^T q_t;
    the heads side by side are normed together (plain weight), multiplied by sigmoid(gate) and projected."""

    def __init__(self, hidden_size: int, num_heads: int, key_dim: int, value_dim: int, decay, norm_eps: float):
        super().__init__()
        if len(decay) != num_heads:
            raise ValueError("one decay per head")
        self.hidden_size, self.num_heads, self.key_dim, self.value_dim = hidden_size, num_heads, key_dim, value_dim
        self.decay_values = tuple(float(d) for d in decay)
        self.norm_eps = float(norm_eps)
        self.qk, self.inner = num_heads * key_dim, num_heads * value_dim
        self.add_child("qkvg", Linear(hidden_size, 2 * self.qk + 2 * self.inner,
                                      parts={"q": self.qk, "k": self.qk, "v": self.inner, "g": self.inner}))
        self.add_param("norm_weight", ParamSpec((self.inner,), init="norm", dtype="float32"))
        self.add_child("o", Linear(self.inner, hidden_size))
        self.decay = None

    def state_need(self):
        return StateNeed((self.num_heads * self.key_dim * self.value_dim,), "float32")

    def finalize(self, device, dtype, max_positions):
        self.decay = torch.tensor(self.decay_values, dtype=torch.float32, device=device)

    def forward(self, x, step, cache, state):
        H, N, P = self.num_heads, self.key_dim, self.value_dim
        rows = self.qkvg.forward(x)                                   # [T, q | k | v | g]
        # silu of q, k and v happens where the recurrence reads them (float32, unrounded)
        y = ops.linear_recurrence(rows[:, : self.qk], rows[:, self.qk: 2 * self.qk], rows[:, 2 * self.qk: 2 * self.qk + self.inner],
                                  state, step.state_slots, step.cu_seqlens, step.q_lens, H, H, N, P, decay=self.decay, silu=True)
        o = ops.gated_rms_norm(y, rows[:, 2 * self.qk + self.inner:], self.norm_weight, self.norm_eps, 1, "sigmoid_behind",
                               rows.dtype)
        return self.o.forward(o, allow_partials=True)


def _log_rates(shape, generator, device):
    """log of decay rates spread over 1..16, the usual start of such a layer."""
    return torch.log(1.0 + 15.0 * torch.rand(shape, generator=generator, dtype=torch.float32, device=device))


def _step_bias(shape, generator, device):
    """Biases whose softplus lies between 0.001 and 0.1."""
    dt = torch.exp(torch.rand(shape, generator=generator, dtype=torch.float32, device=device)
                   * (math.log(0.1) - math.log(0.001)) + math.log(0.001))
    return dt + torch.log(-torch.expm1(-dt))


def _near_one(shape, generator, device):
    return 1.0 + 0.2 * (torch.rand(shape, generator=generator, dtype=torch.float32, device=device) - 0.5)


def _taps(shape, generator, device):
    return (torch.rand(shape, generator=generator, dtype=torch.float32, device=device) - 0.5) * (2.0 / math.sqrt(shape[1]))


@register_part("mixer", "mamba2")
class SelectiveStateSpace(Mixer):
    """One product gives [z | x | B | C | dt]; x, B and C pass a short causal convolution per channel (with
    bias, the last tap is the current token's) and silu; dt = softplus(dt + bias); per head (heads share B and C
    by groups) S_t = exp(-exp(A_log) dt) S_(t-1) + dt B_t x_t^T, y_t = S_t^T C_t + D x_t; y * silu(z), unit root
    mean square over each of `norm_groups` equal parts, a weight, the output product. A request's state row holds
    the heads' matrices and, behind them, the convolution's last taps - 1 inputs per channel."""

    def __init__(self, hidden_size: int, num_heads: int, value_dim: int, state_dim: int, groups: int, taps: int,
                 norm_groups: int, norm_eps: float):
        super().__init__()
        if num_heads % groups or (num_heads * value_dim) % norm_groups or taps < 1:
            raise ValueError("heads must be a multiple of groups, heads * value_dim of norm_groups, taps positive")
        self.hidden_size, self.num_heads, self.value_dim, self.state_dim = hidden_size, num_heads, value_dim, state_dim
        self.groups, self.taps, self.norm_groups, self.norm_eps = groups, taps, norm_groups, float(norm_eps)
        self.inner = num_heads * value_dim
        self.channels = self.inner + 2 * groups * state_dim
        self.add_child("in_proj", Linear(hidden_size, self.inner + self.channels + num_heads))
        self.add_param("conv_weight", ParamSpec((self.channels, taps), init=_taps, dtype="float32"))
        self.add_param("conv_bias", ParamSpec((self.channels,), init="matrix", dtype="float32"))
        self.add_param("dt_bias", ParamSpec((num_heads,), init=_step_bias, dtype="float32"))
        self.add_param("A_log", ParamSpec((num_heads,), init=_log_rates, dtype="float32"))
        self.add_param("D", ParamSpec((num_heads,), init=_near_one, dtype="float32"))
        self.add_param("norm_weight", ParamSpec((self.inner,), init="norm", dtype="float32"))
        self.add_child("o", Linear(self.inner, hidden_size))
        self.matrix_floats = num_heads * state_dim * value_dim
        self.rate = None

    def state_need(self):
        return StateNeed((self.matrix_floats + self.channels * (self.taps - 1),), "float32")

    def finalize(self, device, dtype, max_positions):
        self.rate = torch.exp(self.A_log.float()).contiguous()

    def forward(self, x, step, cache, state):
        H, P, N, G = self.num_heads, self.value_dim, self.state_dim, self.groups
        rows = self.in_proj.forward(x)                                # [T, z | x | B | C | dt]
        xbc = ops.causal_conv(rows[:, self.inner: self.inner + self.channels], self.conv_weight, self.conv_bias,
                              state[:, self.matrix_floats:], step.state_slots, step.cu_seqlens, step.q_lens)
        y = ops.linear_recurrence(xbc[:, self.inner + G * N:], xbc[:, self.inner: self.inner + G * N], xbc[:, : self.inner],
                                  state[:, : self.matrix_floats], step.state_slots, step.cu_seqlens, step.q_lens, H, G, N, P,
                                  dt=rows[:, self.inner + self.channels:], dt_bias=self.dt_bias, rate=self.rate, skip=self.D)
        o = ops.gated_rms_norm(y, rows[:, : self.inner], self.norm_weight, self.norm_eps, self.norm_groups, "silu_before",
                               rows.dtype)
        return self.o.forward(o, allow_partials=True)
