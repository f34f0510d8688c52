"""Element-wise gated recurrences served from the per-sequence state
pool (core/ssm.py)."""

from typing import List

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
