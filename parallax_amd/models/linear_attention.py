"""Recurrent sequence mixers whose state lives in the engine's per-request
slots: gated linear attention (below) and minGRU (class MinGRU).

Gated linear attention (GLA): a matrix-valued recurrent state per head with
a data-dependent decay per key channel,

    S_t = diag(alpha_t) S_(t-1) + k_t v_t^T,     o_t = S_t^T (q_t / sqrt(dk)),
    alpha_t = sigmoid(W_a2 W_a1 h_t + b)^(1/tau),

followed by a per-head RMS norm of o (weight shared by heads), a silu output
gate and the output projection. The state lives in the engine's
LinearStateCache slots in fp32; prompt portions and decode steps both run
ops.gla_recurrence (one HIP kernel, token-serial inside, column-parallel
across the state), so a prompt gives the same state however it is cut.
Decay, gate of the recurrence and the norm are fp32; projections run in the
activation dtype.
"""

from __future__ import annotations

import torch
import torch.nn as nn

from .. import ops
from ..parallel.layers import MergedColumnParallelLinear, RowParallelLinear
from .forward_meta import ForwardMeta


class GatedLinearAttention(nn.Module):
    def __init__(self, hidden_size: int, heads: int, key_dim: int,
                 value_dim: int, tau: float, norm_eps: float,
                 state_layer_idx: int, decay_rank: int = 32):
        super().__init__()
        self.heads, self.dk, self.dv = heads, key_dim, value_dim
        self.tau = float(tau)
        self.eps = norm_eps
        self.state_layer_idx = state_layer_idx
        # one GEMM for q | k | v | output gate
        self.in_proj = MergedColumnParallelLinear(
            hidden_size,
            [heads * key_dim, heads * key_dim, heads * value_dim, heads * value_dim],
        )
        # low-rank decay projection; the rank follows the checkpoint's tensors
        self.decay_down = nn.Parameter(torch.empty(decay_rank, hidden_size),
                                       requires_grad=False)
        self.decay_up = nn.Parameter(torch.empty(heads * key_dim, decay_rank),
                                     requires_grad=False)
        self.decay_bias = nn.Parameter(torch.empty(heads * key_dim),
                                       requires_grad=False)
        self.norm_weight = nn.Parameter(torch.empty(value_dim), requires_grad=False)
        self.o_proj = RowParallelLinear(heads * value_dim, hidden_size)

    def load_decay(self, which: str, t: torch.Tensor) -> None:
        """a1 / a2 carry the decay rank in their shape."""
        name = "decay_down" if which == "a1" else "decay_up"
        setattr(self, name, nn.Parameter(t.clone(), requires_grad=False))

    def forward(self, x: torch.Tensor, meta: ForwardMeta) -> torch.Tensor:
        q, k, v, g = self.in_proj.split_output(self.in_proj(x))
        z = ops.linear(ops.linear(x, self.decay_down), self.decay_up)
        state = meta.linear_cache.recurrent_states[self.state_layer_idx]
        o = ops.gla_recurrence(
            q, k, v, z, self.decay_bias, state, meta.linear_slots,
            meta.query_bounds(), meta.positions, 1.0 / self.tau, self.dk ** -0.5,
        )
        return self.o_proj(ops.gated_rmsnorm(o, g, self.norm_weight, self.eps,
                                             x.dtype))


class MinGRU(nn.Module):
    """minGRU: a gated recurrence over a vector state whose gates read only
    the current token, so the whole portion's gate pre-activations come from
    one GEMM and the recurrence itself is elementwise,

        f_t = sigma(W_z h_t + b_z)            (update gate),
        p_t = W_x h_t + b_x,   c_t = p_t + 1/2 where p_t >= 0, sigma(p_t) below,
        S_t = S_(t-1) + f_t (c_t - S_(t-1)),   o_t = S_t * silu(W_g h_t),

    followed by the output projection. The state [width] lives in the
    engine's LinearStateCache slots in fp32; gates, candidate and state are
    fp32 whatever the activation dtype. Prompt portions and decode steps run
    the same kernel (ops.mingru_scan), token-serial per channel.

    own_proj False: the module has no input projection of its own; a caller
    that merges it with other projections of the same input hands the
    pre-activations [z | u | g] (`proj_sizes` wide) to mix()."""

    def __init__(self, hidden_size: int, width: int, state_layer_idx: int,
                 own_proj: bool = True):
        super().__init__()
        self.width = int(width)
        self.state_layer_idx = state_layer_idx
        self.proj_sizes = [self.width] * 3       # z | u | g
        self.in_proj = MergedColumnParallelLinear(hidden_size, self.proj_sizes) \
            if own_proj else None
        self.z_bias = nn.Parameter(torch.empty(self.width), requires_grad=False)
        self.x_bias = nn.Parameter(torch.empty(self.width), requires_grad=False)
        self.o_proj = RowParallelLinear(self.width, hidden_size)
        self._b32 = None

    def invalidate_constants(self) -> None:
        self._b32 = None

    def mix(self, zug: torch.Tensor, meta: ForwardMeta) -> torch.Tensor:
        """zug [T, 3 * width] (a strided view is fine) -> S_t * silu(g_t)."""
        if self._b32 is None or self._b32[0].device != zug.device:
            self._b32 = (self.z_bias.detach().float().contiguous(),
                         self.x_bias.detach().float().contiguous())
        state = meta.linear_cache.recurrent_states[self.state_layer_idx]
        return ops.mingru_scan(zug, self._b32[0], self._b32[1], state,
                               meta.linear_slots, meta.query_bounds(),
                               meta.positions, self.o_proj.weight.dtype)

    def forward(self, x: torch.Tensor, meta: ForwardMeta) -> torch.Tensor:
        return self.o_proj(self.mix(self.in_proj(x), meta))
