"""Recurrent mixers and token shift served from the per-sequence
state pool (core/ssm.py)."""

import math
from typing import List, Optional

import torch
import torch.nn as nn

from gllm_amd import ops
from gllm_amd.core.ssm import SSMLayerSpec
from gllm_amd.layers.linear import MergedColumnParallelLinear
from gllm_amd.runtime.forward_context import ForwardContext


class MinGRU(nn.Module):
    """minGRU: gates that read only the current token.

        z_t = sigmoid(W_z h_t + b_z)          c_t = g(W_x h_t + b_x)
        S_t = (1 - z_t) S_{t-1} + z_t c_t     g(u) = u + 1/2 (u >= 0),
        out_t = S_t * silu(W_g h_t)                   sigmoid(u) (u < 0)

    z | x | g are one merged projection (the biases of z and x ride on
    its bias, zero for g); gates, candidate and the state [slots, width]
    are fp32. The read-out projection is left to the caller, who may
    have the result written (scaled) into a column block of a wider
    buffer to share one output GEMM with a sibling mixer.
    """

    def __init__(self, hidden: int, width: int, ssm_layer_id: int,
                 params_dtype=None, own_proj: bool = True):
        """``own_proj`` False: the caller computes z | x | g inside a
        projection of its own (columns sized ``self.sizes``) and calls
        ``forward_projected``."""
        super().__init__()
        self.width = width
        self.ssm_layer_id = ssm_layer_id
        self.sizes: List[int] = [width, width, width]
        if own_proj:
            self.in_proj = MergedColumnParallelLinear(
                hidden, self.sizes, bias=True, params_dtype=params_dtype)
            self.in_proj.bias.data.zero_()
        else:
            self.in_proj = None
        self._ones = None

    def spec(self) -> SSMLayerSpec:
        return SSMLayerSpec(0, 1, 1, 1, self.width,
                            state_shape=(self.width,))

    def forward(self, h: torch.Tensor, fctx: ForwardContext,
                out: torch.Tensor = None, scale: float = 1.0):
        """h [T, hidden] -> scale * S_t * silu(gate) [T, width]."""
        proj = self.in_proj(h)
        return self.forward_projected(proj[:, :2 * self.width],
                                      proj[:, 2 * self.width:], fctx, out,
                                      scale)

    def forward_projected(self, zx: torch.Tensor, gp: torch.Tensor,
                          fctx: ForwardContext, out: torch.Tensor = None,
                          scale: float = 1.0):
        """zx [T, 2*width] = z | x pre-activations (biases added), gp
        [T, width] gate logits; row views of a wider projection are
        fine. ``out`` may be a column block of a wider buffer."""
        T = zx.shape[0]
        if fctx.is_profile_run or fctx.ssm_pool is None:
            if out is not None:
                out.zero_()
                return out
            return zx.new_zeros(T, self.width)
        if fctx.ssm_slots_dev is not None:
            # captured decode bucket: every row continues carried state
            slots = fctx.ssm_slots_dev[:T]
            if self._ones is None or self._ones.numel() < T \
                    or self._ones.device != zx.device:
                self._ones = torch.ones(max(T, 1024), dtype=torch.int32,
                                        device=zx.device)
            init = self._ones[:T]
        else:
            slots, init = fctx.ssm_slots_t, fctx.ssm_has_init_t
        return ops.mingru_varlen(
            zx, gp, fctx.ssm_pool.ssm_state[self.ssm_layer_id], slots, init,
            fctx.query_start_loc, scale, fctx.max_query_len, out)


_ONES = {}


def state_rows(fctx: ForwardContext, T: int, device):
    """(slots, carried-state flags) of a batch for the ragged state
    kernels. Inside a captured decode bucket every row is a one-token
    step on carried state and the slots come from the runner's
    persistent buffer (padding rows work on the pool's scratch slot)."""
    if fctx.ssm_slots_dev is not None:
        ones = _ONES.get(device)
        if ones is None or ones.numel() < T:
            ones = _ONES[device] = torch.ones(
                max(T, 1024), dtype=torch.int32, device=device)
        return fctx.ssm_slots_dev[:T], ones[:T]
    return fctx.ssm_slots_t, fctx.ssm_has_init_t


class TokenShift(nn.Module):
    """h_t <- h_t + (h_(t-1) - h_t) * mu, per channel, h_(t-1) being the
    previous token's row as it came in (zeros ahead of a sequence's
    first token). The last incoming row of every sequence lives in the
    state pool (``shift_state[ssm_layer_id]``), so prompt portions and
    decode steps continue each other."""

    def __init__(self, width: int, ssm_layer_id: int, params_dtype=None):
        super().__init__()
        dtype = params_dtype or torch.get_default_dtype()
        self.ssm_layer_id = ssm_layer_id
        self.mu = nn.Parameter(torch.zeros(width, dtype=dtype),
                               requires_grad=False)

    def forward(self, h: torch.Tensor, fctx: ForwardContext,
                ssm_layer_id: Optional[int] = None) -> torch.Tensor:
        if fctx.is_profile_run or fctx.ssm_pool is None:
            return h
        sid = self.ssm_layer_id if ssm_layer_id is None else ssm_layer_id
        slots, init = state_rows(fctx, h.shape[0], h.device)
        return ops.token_shift(h, self.mu, fctx.ssm_pool.shift_state[sid],
                               slots, init, fctx.query_start_loc,
                               fctx.max_query_len)


class GeneralDeltaRule(nn.Module):
    """Delta rule with a decay per key channel and a removal rate per
    key channel, ``heads`` heads of key size ``dim`` and value size
    ``vdim``:

        w_t = exp(-decay_scale * sigmoid(w_logit_t + w0))
        a_t = sigmoid(a_logit_t)       u_t = k_t / sqrt(|k_t|^2 + 1e-6)
        S_t = diag(w_t) S_(t-1) - (a_t u_t)(u_t^T S_(t-1)) + k_t v_t^T
        o_t = S_t^T r_t

    and a read-out scale * o / rms(o) * norm_weight * sigmoid(gate) per
    head (``norm_weight`` [heads * vdim]: every head has its own). The
    caller owns the projections (r, k, v, the two logit rows, the gate;
    row views of a merged projection are fine); decay, removal rate,
    unit key and the state [slots, heads, dim, vdim] are fp32.
    """

    def __init__(self, heads: int, dim: int, vdim: int, eps: float,
                 ssm_layer_id: int, decay_scale: float = math.exp(-0.5),
                 params_dtype=None):
        super().__init__()
        dtype = params_dtype or torch.get_default_dtype()
        self.heads, self.dim, self.vdim = heads, dim, vdim
        self.eps = eps
        self.decay_scale = float(decay_scale)
        self.ssm_layer_id = ssm_layer_id
        self.w0 = nn.Parameter(torch.zeros(heads * dim, dtype=dtype),
                               requires_grad=False)
        self.norm_weight = nn.Parameter(
            torch.ones(heads * vdim, dtype=dtype), requires_grad=False)

    def spec(self, conv_dim: int = 0, conv_kernel: int = 1,
             shift_dim: int = 0) -> SSMLayerSpec:
        """Pool geometry of one run of the layer; a sibling's short
        convolution and a token shift ride on the same entry."""
        return SSMLayerSpec(conv_dim, conv_kernel, self.heads, self.dim,
                            self.vdim, layout="kv", shift_dim=shift_dim)

    def forward(self, r, k, v, w_logit, a_logit, gate,
                fctx: ForwardContext, out: torch.Tensor = None,
                scale: float = 1.0, ssm_layer_id: Optional[int] = None):
        T = r.shape[0]
        if fctx.is_profile_run or fctx.ssm_pool is None:
            if out is not None:
                out.zero_()
                return out
            return r.new_zeros(T, self.heads * self.vdim)
        sid = self.ssm_layer_id if ssm_layer_id is None else ssm_layer_id
        slots, init = state_rows(fctx, T, r.device)
        o = ops.general_delta_rule(
            r, k, v, w_logit, a_logit, self.w0, self.decay_scale,
            fctx.ssm_pool.ssm_state[sid], slots, init,
            fctx.query_start_loc, fctx.max_query_len)
        return ops.rms_gate(o, gate, self.norm_weight, self.heads, self.eps,
                            r.dtype, gate="sigmoid", scale=scale, out=out)
