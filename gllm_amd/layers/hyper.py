"""Hyper-connections: a residual made of several parallel streams.

The residual of every token is ``streams`` fp32 vectors x_1..x_S (all
equal to the embedding at the start, summed at the end). A sublayer
reads one learned mixture of them and its result is written back into
every stream while the streams are mixed among themselves:

    u   = sum_s in[s] x_s
    y   = sublayer(norm(u))
    x_t = sum_s mix[s, t] x_s + out[t] y        (all t from the old x)

``norm`` is an RMS norm whose gain is one number. S = 1 with in = out =
mix = 1 is the ordinary pre-norm residual, which is how a model without
the extra tensors runs through the same code.

Streams are held as one tensor [S, T, W]. ``HyperConnection.write``
takes the NEXT sublayer's connection and fuses its read into the same
launch (ops.hyper_streams), so a sublayer boundary costs one kernel.
"""

from typing import Optional

import torch
import torch.nn as nn

from gllm_amd import ops


class ScalarRMSNorm(nn.Module):
    """x / sqrt(mean(x^2) + eps) * g with a single learned number g."""

    def __init__(self, eps: float):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(1, dtype=torch.float32),
                                   requires_grad=False)
        self.eps = eps

    def load(self, w: torch.Tensor) -> None:
        assert w.numel() == 1, tuple(w.shape)
        self.weight.data.copy_(w.reshape(1).float())


class HyperConnection(nn.Module):
    """One sublayer's read weights, write weights and stream mix, with
    the scalar-gain norm the sublayer reads through. Parameters are fp32
    (the stream arithmetic is fp32 whatever the model dtype is)."""

    def __init__(self, streams: int, eps: float):
        super().__init__()
        S = streams
        self.streams = S
        self.norm = ScalarRMSNorm(eps)
        self.in_w = nn.Parameter(torch.ones(S, dtype=torch.float32),
                                 requires_grad=False)
        self.out_w = nn.Parameter(torch.ones(S, dtype=torch.float32),
                                  requires_grad=False)
        self.mix = nn.Parameter(torch.eye(S, dtype=torch.float32),
                                requires_grad=False)

    def _read_args(self):
        return (self.in_w, self.norm.weight, self.norm.eps)

    def read(self, xs: torch.Tensor, dtype) -> torch.Tensor:
        """norm(sum_s in[s] x_s) in the model dtype."""
        return ops.hyper_streams(xs, read=self._read_args(), dtype=dtype)

    def write(self, xs: torch.Tensor, y: torch.Tensor,
              nxt: Optional["HyperConnection"] = None,
              y2: Optional[torch.Tensor] = None,
              gate: Optional[torch.Tensor] = None):
        """Write y (+ sigmoid(gate) * y2, one gate logit per row) back
        into the streams in place; with ``nxt`` also return what the
        next sublayer reads."""
        return ops.hyper_streams(
            xs, y, y2, gate, self.mix, self.out_w,
            read=None if nxt is None else nxt._read_args(), dtype=y.dtype)


def sum_reader(streams: int, eps: float) -> HyperConnection:
    """The read at the end of the stack: the plain sum of the streams
    through the model's last norm."""
    return HyperConnection(streams, eps)
