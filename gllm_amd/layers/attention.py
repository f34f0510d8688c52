"""Paged attention layer (reference: layers/attention.py FlashAttention).

One module instance per decoder layer; forward stores new K/V into the
paged cache (HIP scatter kernel) then runs the varlen paged-attention
kernel family (prefill MFMA kernel / split-KV decode kernel, dispatched
in ops.paged_attention).
"""

from typing import Optional

import torch
import torch.nn as nn

from gllm_amd import ops
from gllm_amd.runtime.forward_context import ForwardContext


class Attention(nn.Module):
    def __init__(self, layer_idx: int, num_heads: int, num_kv_heads: int,
                 head_dim: int, scale: float, sliding_window: int = 0):
        super().__init__()
        self.layer_idx = layer_idx       # LOCAL layer index on this PP stage
        self.num_heads = num_heads       # per TP rank
        self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim
        self.scale = scale
        self.sliding_window = sliding_window

    def forward(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                fctx: ForwardContext) -> torch.Tensor:
        T = q.shape[0]
        q = q.unflatten(-1, (self.num_heads, self.head_dim))
        k = k.unflatten(-1, (self.num_kv_heads, self.head_dim))
        v = v.unflatten(-1, (self.num_kv_heads, self.head_dim))
        if fctx.is_profile_run:
            # Peak-memory profile pass runs before the KV cache exists
            # (reference layers/attention.py:112-116): skip attention math,
            # return a same-shape tensor.
            return q.reshape(T, -1)
        k_cache = fctx.k_caches[self.layer_idx]
        v_cache = fctx.v_caches[self.layer_idx]
        ops.reshape_and_cache(k, v, k_cache, v_cache, fctx.slot_mapping)
        out = ops.paged_attention(
            q, k_cache, v_cache, fctx.block_table, fctx.seq_lens,
            fctx.query_start_loc, self.scale,
            max_query_len=fctx.max_query_len,
            sliding_window=self.sliding_window)
        return out.reshape(T, -1)


class WindowAttention(nn.Module):
    """Paged attention with a sliding window that keeps the first tokens
    visible, an optional softmax sink and a fused output gate.

    * per-head query/key size ``head_dim`` and value size ``v_head_dim``
      may differ; any GQA ratio
    * q/k get a per-head RMS norm (plain weights ``q_norm``/``k_norm``)
      and an interleaved-pair rotary (``rotary``: layers.rotary
      .PairRotary or None) inside one fused kernel that also stores k, v
      in the paged cache
    * position i sees j <= i with i - j < ``window`` or j < ``keep_first``
      (window 0 = plain causal)
    * ``sink``: softmax denominator 1 + sum exp(s); ``sink="learned"``:
      exp(sinks[h]) + sum exp(s) with the fp32 parameter ``sinks`` [H]
    * ``qk_norm`` False: q and k are rotated only (no per-head norm)
    * ``softcap`` > 0: scores become cap * tanh(score / cap)
    * ``value_rotary`` (a PairRotary over all of ``v_head_dim``): the
      value of position j enters the cache turned by j, and each head's
      weighted sum at position i is turned back by i, so what a query
      receives from a key depends on their distance only
    * ``norm_span``: q (and k) get ONE RMS over all heads of the token
      with weights that cover the whole row ([H*D], [G*D]) instead of a
      norm per head; ``value_unit_norm``: every value head enters the
      cache divided by its RMS (eps, no weight). A ``rotary`` with
      ``half_layout`` pairs dimension i with i + rot_dims/2
    * ``kv_source``: cache index of ANOTHER layer whose keys and values
      this layer attends over; such a layer owns no k/v tensors and
      stores nothing (``owns_kv`` False)

    Everything runs in the dtype of q (bf16 or fp32) with fp32 scores.
    """

    def __init__(self, layer_idx: int, num_heads: int, num_kv_heads: int,
                 head_dim: int, v_head_dim: int, scale: float, eps: float,
                 window: int = 0, keep_first: int = 0, sink=False,
                 rotary: Optional[nn.Module] = None, owns_kv: bool = True,
                 params_dtype=None, qk_norm: bool = True,
                 softcap: float = 0.0,
                 value_rotary: Optional[nn.Module] = None,
                 norm_span: bool = False, value_unit_norm: bool = False):
        super().__init__()
        dtype = params_dtype or torch.get_default_dtype()
        self.norm_span = norm_span
        self.value_unit_norm = value_unit_norm
        self.layer_idx = layer_idx       # cache this layer reads
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim
        self.v_head_dim = v_head_dim
        self.scale = scale
        self.eps = eps
        self.window = window
        self.keep_first = keep_first
        self.sink = bool(sink) and sink != "learned"
        self.rotary = rotary
        self.owns_kv = owns_kv
        self.qk_norm = qk_norm
        self.softcap = float(softcap or 0.0)
        self.value_rotary = value_rotary
        if value_rotary is not None:
            assert value_rotary.rot_dims == v_head_dim
        if qk_norm:
            nq = num_heads * head_dim if norm_span else head_dim
            nk = num_kv_heads * head_dim if norm_span else head_dim
            self.q_norm = nn.Parameter(torch.ones(nq, dtype=dtype),
                                       requires_grad=False)
            if owns_kv:
                self.k_norm = nn.Parameter(
                    torch.ones(nk, dtype=dtype), requires_grad=False)
        else:
            self.q_norm = self.k_norm = None
        if sink == "learned":
            self.sinks = nn.Parameter(
                torch.zeros(num_heads, dtype=torch.float32),
                requires_grad=False)
        else:
            self.sinks = None
        self._no_rot = None

    def _freqs(self, device):
        if self.rotary is not None:
            return self.rotary.freqs, self.rotary.mag, self.rotary.rot_dims
        if self._no_rot is None or self._no_rot.device != device:
            self._no_rot = torch.zeros(1, dtype=torch.float64, device=device)
        return self._no_rot, 1.0, 0

    def forward(self, q: torch.Tensor, k: Optional[torch.Tensor],
                v: Optional[torch.Tensor], gate: Optional[torch.Tensor],
                fctx: ForwardContext, out: Optional[torch.Tensor] = None,
                out_scale: float = 1.0,
                layer_idx: Optional[int] = None) -> torch.Tensor:
        """q [T, H*D], k [T, G*D], v [T, G*Dv], gate [T, H*Dv] (row
        views of a merged projection are fine). Returns [T, H*Dv],
        multiplied by ``out_scale`` and written into ``out`` (which may
        be a column block of a wider buffer) when those are given.
        ``layer_idx`` overrides the cache index (a layer that runs
        several times keeps one cache per run)."""
        T = q.shape[0]
        idx = self.layer_idx if layer_idx is None else layer_idx
        if fctx.is_profile_run:
            if out is not None:
                out.zero_()
                return out
            return q.new_zeros(T, self.num_heads * self.v_head_dim)
        k_cache = fctx.k_caches[idx]
        v_cache = fctx.v_caches[idx]
        freqs, mag, rot_dims = self._freqs(q.device)
        half = bool(getattr(self.rotary, "half_layout", False))
        vrot = self.value_rotary
        vfreqs = vrot.freqs if vrot is not None else None
        q_out = None
        if self.norm_span:
            # every head reads the whole incoming row: queries land in
            # a buffer of their own
            q_out = torch.empty(T, self.num_heads * self.head_dim,
                                dtype=q.dtype, device=q.device)
        if self.owns_kv:
            ops.qk_norm_rope_store(
                q, k, v, self.q_norm, self.k_norm, fctx.positions,
                fctx.slot_mapping, freqs, mag, rot_dims, k_cache, v_cache,
                self.num_heads, self.num_kv_heads, self.head_dim,
                self.v_head_dim, self.eps, half_layout=half,
                do_norm=self.qk_norm, v_freqs=vfreqs,
                norm_span=self.norm_span, v_unit=self.value_unit_norm,
                q_out=q_out)
        else:
            ops.qk_norm_rope_store(
                q, None, None, self.q_norm, None, fctx.positions,
                fctx.slot_mapping, freqs, mag, rot_dims, None, None,
                self.num_heads, self.num_kv_heads, self.head_dim,
                self.v_head_dim, self.eps, half_layout=half,
                do_norm=self.qk_norm, norm_span=self.norm_span,
                q_out=q_out)
        if q_out is not None:
            q = q_out
        direct = out if (vrot is None and out_scale == 1.0) else None
        o = ops.window_attention(
            q, gate, k_cache, v_cache, fctx.block_table, fctx.seq_lens,
            fctx.query_start_loc, self.scale, self.window,
            self.keep_first, self.sink, fctx.max_query_len,
            sinks=self.sinks, softcap=self.softcap, out=direct)
        if direct is not None:
            return out
        if vrot is not None:
            # turn every head's sum back by the query's own position
            return ops.rotate_scale_rows(
                o, fctx.positions, vfreqs, self.num_heads, self.v_head_dim,
                -1.0, out_scale, out=out)
        if out is not None:
            out.copy_(o if out_scale == 1.0 else o * out_scale)
            return out
        return o if out_scale == 1.0 else o * out_scale


class TalkingHeadsAttention(nn.Module):
    """Paged causal attention whose heads talk before the softmax.

    * keys double as values: the cache of this layer holds the
      normalised, rotated keys (K side) and the keys as projected (V
      side); there is no value projection
    * q and k are rotated (``rotary``: layers.rotary.HalfRotary /
      PairRotary or None) and then brought to unit RMS per head, with no
      learned weight, inside one fused kernel that also writes the cache
    * the H per-head score planes scale * q_g . k are mixed by ``talk``
      [H, H] (s'_h = sum_g talk[h, g] s_g) before masking and softmax
    * ``sink`` [H]: exp(sink_h) joins head h's softmax denominator

    ``talk`` and ``sink`` are fp32 parameters (scores and softmax run in
    fp32 whatever the model dtype is). Any GQA ratio, any head size.
    """

    def __init__(self, layer_idx: int, num_heads: int, num_kv_heads: int,
                 head_dim: int, scale: float, eps: float,
                 rotary: Optional[nn.Module] = None, sink: bool = True):
        super().__init__()
        assert num_heads % num_kv_heads == 0
        self.layer_idx = layer_idx
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim
        self.scale = scale
        self.eps = eps
        self.rotary = rotary
        self.talk = nn.Parameter(torch.eye(num_heads, dtype=torch.float32),
                                 requires_grad=False)
        if sink:
            self.sink = nn.Parameter(
                torch.zeros(num_heads, dtype=torch.float32),
                requires_grad=False)
        else:
            self.register_parameter("sink", None)
        self._no_rot = None

    def _freqs(self, device):
        r = self.rotary
        if r is not None:
            return r.freqs, r.mag, r.rot_dims, \
                bool(getattr(r, "half_layout", False))
        if self._no_rot is None or self._no_rot.device != device:
            self._no_rot = torch.zeros(1, dtype=torch.float64, device=device)
        return self._no_rot, 1.0, 0, False

    def forward(self, q: torch.Tensor, k: torch.Tensor,
                fctx: ForwardContext,
                layer_idx: Optional[int] = None) -> torch.Tensor:
        """q [T, H*D], k [T, G*D] (row views of a merged projection are
        fine). ``layer_idx`` overrides the cache index (a layer that
        runs several times keeps one cache per run). Returns [T, H*D]."""
        T = q.shape[0]
        H, G, D = self.num_heads, self.num_kv_heads, self.head_dim
        if fctx.is_profile_run:
            return q.new_zeros(T, H * D)
        idx = self.layer_idx if layer_idx is None else layer_idx
        k_cache, v_cache = fctx.k_caches[idx], fctx.v_caches[idx]
        freqs, mag, rot_dims, half = self._freqs(q.device)
        ops.qk_norm_rope_store(
            q, k, k, None, None, fctx.positions, fctx.slot_mapping, freqs,
            mag, rot_dims, k_cache, v_cache, H, G, D, D, self.eps,
            half_layout=half, norm_last=True)
        return ops.talking_attention(
            q, k_cache, v_cache, fctx.block_table, fctx.seq_lens,
            fctx.query_start_loc, self.scale, self.talk, self.sink,
            fctx.max_query_len)


class LatentAttention(nn.Module):
    """Causal attention whose keys and values are up-projections of one
    cached low-rank latent per token, without positions.

        c_t   = RMSnorm(W_dkv h_t)                  (the only cached row)
        k_j,h = W_uk,h c_j      v_j,h = W_uv,h c_j
        s     = scale * q_i,h . k_j,h,  softmax over j <= i

    The up-projections are never applied to the cache: the query is
    carried into the latent space (q~ = W_uk,h^T q, so q~ . c = q . k),
    attention runs over the latent rows themselves as one shared
    key/value head, and the per-head weighted latent is brought to the
    value space afterwards (W_uv,h applied to the sum). The cache of the
    layer is ``[pages, page, 1, rank]`` and serves as key and value
    cache at once.

    ``owns_kv`` False: the layer has no W_dkv and attends over the
    latent another layer cached (``layer_idx`` names that cache), with
    up-projections of its own.

    ``w_uk`` [H, D, rank] and ``w_uv`` [H, Dv, rank] are parameters of
    this module; the down projections and their norms live in the
    caller's merged projection.
    """

    def __init__(self, layer_idx: int, num_heads: int, head_dim: int,
                 v_head_dim: int, rank: int, scale: float, eps: float,
                 owns_kv: bool = True, params_dtype=None):
        super().__init__()
        dtype = params_dtype or torch.get_default_dtype()
        self.layer_idx = layer_idx
        self.num_heads = num_heads
        self.head_dim = head_dim
        self.v_head_dim = v_head_dim
        self.rank = rank
        self.scale = scale
        self.eps = eps
        self.owns_kv = owns_kv
        self.w_uk = nn.Parameter(
            torch.empty(num_heads, head_dim, rank, dtype=dtype),
            requires_grad=False)
        self.w_uv = nn.Parameter(
            torch.empty(num_heads, v_head_dim, rank, dtype=dtype),
            requires_grad=False)
        if owns_kv:
            self.kv_norm = nn.Parameter(torch.ones(rank, dtype=dtype),
                                        requires_grad=False)

    def forward(self, q: torch.Tensor, ckv: Optional[torch.Tensor],
                fctx: ForwardContext) -> torch.Tensor:
        """q [T, H*D]; ckv [T, rank] = W_dkv h before its norm (None for
        a layer that reads another layer's latent). Returns [T, H*Dv]."""
        T = q.shape[0]
        H, D, Dv, R = self.num_heads, self.head_dim, self.v_head_dim, \
            self.rank
        if fctx.is_profile_run:
            return q.new_zeros(T, H * Dv)
        cache = fctx.k_caches[self.layer_idx]
        if self.owns_kv:
            ops.rms_weight_store(ckv, self.kv_norm, self.eps, cache,
                                 fctx.slot_mapping)
        # q~[t, h] = W_uk,h^T q[t, h]
        q_lat = torch.bmm(q.reshape(T, H, D).transpose(0, 1), self.w_uk)
        q_lat = q_lat.transpose(0, 1).reshape(T, H * R)
        o_lat = ops.window_attention(
            q_lat, None, cache, cache, fctx.block_table, fctx.seq_lens,
            fctx.query_start_loc, self.scale, 0, 0, False,
            fctx.max_query_len)
        # o[t, h] = W_uv,h o~[t, h]
        o = torch.bmm(o_lat.reshape(T, H, R).transpose(0, 1),
                      self.w_uv.transpose(1, 2))
        return o.transpose(0, 1).reshape(T, H * Dv)
