"""RMSNorm layers over the fused HIP kernels (reference: layers/layernorm.py)."""

from typing import Optional

import torch
import torch.nn as nn

from gllm_amd import ops


class RMSNorm(nn.Module):
    def __init__(self, hidden_size: int, eps: float = 1e-6):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(hidden_size))
        self.eps = eps

    def forward(self, x: torch.Tensor,
                residual: Optional[torch.Tensor] = None):
        if residual is not None:
            return ops.fused_add_rmsnorm(x, residual, self.weight, self.eps)
        return ops.rmsnorm(x, self.weight, self.eps)


class GemmaRMSNorm(nn.Module):
    """(1 + w) convention (Qwen3.5/Gemma checkpoints store w - 1).

    The effective scale (1 + w) is cached after load so the hot path
    runs the same fused add+rmsnorm kernel as RMSNorm."""

    def __init__(self, hidden_size: int, eps: float = 1e-6):
        super().__init__()
        self.weight = nn.Parameter(torch.zeros(hidden_size))
        self.eps = eps
        self._w1 = None

    def _scale(self):
        if self._w1 is None or self._w1.device != self.weight.device:
            self._w1 = (self.weight + 1.0).contiguous()
        return self._w1

    def forward(self, x: torch.Tensor,
                residual: Optional[torch.Tensor] = None):
        if residual is not None:
            return ops.fused_add_rmsnorm(x, residual, self._scale(),
                                         self.eps)
        return ops.rmsnorm(x, self._scale(), self.eps)


class LayerNorm(nn.Module):
    """LayerNorm with weight and (optional) bias over an fp32 residual
    stream.

    Sandwich-norm decoders (a norm before and after every sublayer) keep
    the stream in fp32 while sublayers run in the model dtype:

    * ``norm(x)``                       h = LN(x), x fp32 -> model dtype
    * ``norm.add_into(x, y, nxt)``      x += LN(y) in place and, when
      ``nxt`` (the next sublayer's pre-norm) is given, returns nxt(x) —
      one fused launch per boundary (ops.residual_layernorm)
    * ``norm.add_into(x, y, nxt, gate=g)``  the same with the sublayer
      result gated first: x += LN(y * sigmoid(g))

    The bias parameter is named ``bias`` (None with ``bias=False``);
    checkpoints that store it under another name map it in the model's
    load_weights.
    """

    def __init__(self, hidden_size: int, eps: float = 1e-5,
                 params_dtype=None, bias: bool = True):
        super().__init__()
        dtype = params_dtype or torch.get_default_dtype()
        self.weight = nn.Parameter(torch.ones(hidden_size, dtype=dtype),
                                   requires_grad=False)
        if bias:
            self.bias = nn.Parameter(torch.zeros(hidden_size, dtype=dtype),
                                     requires_grad=False)
        else:
            self.register_parameter("bias", None)
        self.eps = eps
        self._w32 = None

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return ops.layernorm_f32(x, self.weight, self.bias, self.eps,
                                 self.weight.dtype)

    def forward_f32(self, x: torch.Tensor) -> torch.Tensor:
        """LN(x) kept in fp32 (a norm whose result IS the residual
        stream, e.g. right after the embedding)."""
        if self.weight.dtype == torch.float32:
            return self.forward(x)
        if self._w32 is None or self._w32[0].device != x.device:
            self._w32 = (self.weight.float(), None if self.bias is None
                         else self.bias.float())
        return ops.layernorm_f32(x, self._w32[0], self._w32[1], self.eps,
                                 torch.float32)

    def add_into(self, x: torch.Tensor, y: torch.Tensor,
                 nxt: Optional["LayerNorm"] = None,
                 gate: Optional[torch.Tensor] = None):
        pre = (nxt.weight, nxt.bias) if nxt is not None else None
        return ops.residual_layernorm(x, y, self.weight, self.bias,
                                      self.eps, pre, gate)


class StreamRMSNorm(nn.Module):
    """RMS norm (plain weight, eps inside the root) over an fp32
    residual stream, for decoders that norm before AND after every
    sublayer and add the normed result times a fixed multiplier:

    * ``norm(x)``                          h = RMSnorm(x) * w, model dtype
    * ``norm.add_into(x, y, nxt, mult)``   x += mult * RMSnorm(y) * w in
      place and, with ``nxt`` (the next sublayer's pre-norm), returns
      nxt(x): one launch per boundary (ops.stream_rmsnorm)
    * ``y2``: the norm sees y + y2 (a routed and a shared result);
      ``y_scale``: it sees y_scale * (y + y2), the product formed in
      fp32; ``add`` (fp32 [width]): added to every row of x after the
      sublayer result and before ``nxt`` reads it
    """

    def __init__(self, hidden_size: int, eps: float = 1e-5,
                 params_dtype=None):
        super().__init__()
        dtype = params_dtype or torch.get_default_dtype()
        self.weight = nn.Parameter(torch.ones(hidden_size, dtype=dtype),
                                   requires_grad=False)
        self.eps = eps

    def forward(self, x: torch.Tensor,
                add: Optional[torch.Tensor] = None) -> torch.Tensor:
        return ops.stream_rmsnorm(x, None, None, self.eps, add=add,
                                  pre_w=self.weight)

    def add_into(self, x: torch.Tensor, y: torch.Tensor,
                 nxt: Optional["StreamRMSNorm"] = None, mult: float = 1.0,
                 y_scale: float = 1.0, y2: Optional[torch.Tensor] = None,
                 add: Optional[torch.Tensor] = None):
        return ops.stream_rmsnorm(
            x, y, self.weight, self.eps, mult, y_scale, y2, add,
            nxt.weight if nxt is not None else None)
