"""Gopetar: a config-driven decoder over a multi-stream residual.

``config.layers`` describes every layer on its own (mixer type, mixer
sizes, feed-forward), so sizes may differ from layer to layer and the
layers come in any order.

* stream: ``streams`` fp32 copies of embed[token] * embedding.scale,
  read and written through hyper-connections (layers/hyper.py): every
  sublayer reads a learned mixture of the streams through an RMS norm
  with a one-number gain and writes its result back into all of them;
  the logits come from the norm of their sum
* mixer ``parallel``: two mixers on the same input, their results
  weighted and added —
  left: GQA with biased q/k/v, interleaved-pair rotary on the first
  ``rot.dims`` dims (wavelength-dependent frequency scaling), values
  rotated by their own position over all of vdim and the head sums
  rotated back by the query's, tanh-capped scores, a sliding window
  and a learned per-head sink in the softmax denominator;
  right: minGRU (layers/recurrent.py) with an fp32 state per sequence
* mixer ``latent_attention``: causal attention without positions whose
  keys and values are up-projections of a cached normed low-rank
  latent, queries through a normed latent of their own; a layer with
  ``kv_from: j`` attends over layer j's cached latent with its own
  up-projections
* feed-forward: top-k-of-logits mixture of clamped-SwiGLU experts
  (fp32 router, softmax over the chosen logits) plus a shared expert
  gated per token by sigmoid(w_sg . h)

Framework mapping: one merged input projection per mixer (q | k | v |
z | x | g, dq | dkv) and one output GEMM for the two parallel branches
(their scaled results are written side by side, layers/linear.py),
WindowAttention / LatentAttention (layers/attention.py), PairRotary
(layers/rotary.py), MinGRU over the state pool (core/ssm.py), FusedMoE
with ``activation="swiglu_clamp"`` (layers/moe/layer.py), the paged KV
pool with per-layer shapes (core/kv_cache.py; a latent layer's value
cache is its key cache). Prompt portions and decode tokens of a mixed
batch run through the same ragged kernels.
"""

from typing import Iterable, List, Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from gllm_amd import ops
from gllm_amd.core.ssm import SSMLayerSpec, SSMSpec
from gllm_amd.layers.attention import LatentAttention, WindowAttention
from gllm_amd.layers.embedding import ParallelLMHead, VocabParallelEmbedding
from gllm_amd.layers.hyper import HyperConnection, sum_reader
from gllm_amd.layers.linear import (MergedColumnParallelLinear,
                                    ReplicatedLinear, RowParallelLinear)
from gllm_amd.layers.moe.layer import FusedMoE
from gllm_amd.layers.recurrent import MinGRU
from gllm_amd.layers.rotary import PairRotary
from gllm_amd.runtime.forward_context import ForwardContext

# sigmoid slope of the expert activation g * sigmoid(1.702 g) * (u + 1)
EXPERT_ALPHA = 1.702


def _get(d, key, default=None):
    """config.json sub-objects arrive as dicts (or namespaces)."""
    if d is None:
        return default
    if isinstance(d, dict):
        return d.get(key, default)
    return getattr(d, key, default)


class ParallelMixer(nn.Module):
    """Windowed sink attention beside a minGRU: one input GEMM
    (q | k | v | z | x | g), one output GEMM over [left_scale * heads |
    right_scale * recurrence read-out]."""

    def __init__(self, width: int, m, eps: float, kv_index: int,
                 ssm_layer_id: int, dtype):
        super().__init__()
        left, right = _get(m, "left"), _get(m, "right")
        H, G = int(_get(left, "heads")), int(_get(left, "kv_heads"))
        D, Dv = int(_get(left, "dim")), int(_get(left, "vdim"))
        C = int(_get(right, "width"))
        self.left_scale = float(_get(m, "left_scale", 1.0))
        self.right_scale = float(_get(m, "right_scale", 1.0))
        self.attn_sizes = [H * D, G * D, G * Dv]
        self.gru = MinGRU(width, C, ssm_layer_id, params_dtype=dtype,
                          own_proj=False)
        self.sizes = self.attn_sizes + self.gru.sizes
        self.in_proj = MergedColumnParallelLinear(width, self.sizes,
                                                  bias=True,
                                                  params_dtype=dtype)
        self.in_proj.bias.data.zero_()
        self.heads_out = H * Dv
        self.out_proj = RowParallelLinear(H * Dv + C, width,
                                          params_dtype=dtype)
        rot = _get(left, "rot")
        rotary = vrot = None
        if rot:
            if int(_get(rot, "dims", 0) or 0) > 0:
                rotary = PairRotary(int(_get(rot, "dims")),
                                    float(_get(rot, "base")),
                                    _get(rot, "scaling"))
            vrot = PairRotary(Dv, float(_get(rot, "base")))
        mask = _get(left, "mask")
        self.attn = WindowAttention(
            kv_index, H, G, D, Dv, float(_get(left, "scale")), eps,
            window=int(_get(mask, "size", 0) or 0), sink="learned",
            rotary=rotary, params_dtype=dtype, qk_norm=False,
            softcap=float(_get(left, "softcap", 0.0) or 0.0),
            value_rotary=vrot)

    SHARDS = {("left", "q"): 0, ("left", "k"): 1, ("left", "v"): 2,
              ("right", "z"): 3, ("right", "x"): 4, ("right", "g"): 5}

    def forward(self, h: torch.Tensor, fctx: ForwardContext):
        proj = self.in_proj(h)
        na = sum(self.attn_sizes)
        q, k, v = proj[:, :na].split(self.attn_sizes, dim=-1)
        C = self.gru.width
        zx, gp = proj[:, na:na + 2 * C], proj[:, na + 2 * C:]
        both = torch.empty(h.shape[0], self.heads_out + C, dtype=h.dtype,
                           device=h.device)
        self.attn(q, k, v, None, fctx, out=both[:, :self.heads_out],
                  out_scale=self.left_scale)
        self.gru.forward_projected(zx, gp, fctx,
                                   out=both[:, self.heads_out:],
                                   scale=self.right_scale)
        return self.out_proj(both)


class LatentMixer(nn.Module):
    """dq | dkv in one projection, normed query latent -> queries,
    attention over the cached normed kv latent, output projection."""

    def __init__(self, width: int, m, eps: float, kv_index: int,
                 owns_kv: bool, dtype):
        super().__init__()
        H, D, Dv = int(_get(m, "heads")), int(_get(m, "dim")), \
            int(_get(m, "vdim"))
        self.q_rank, self.kv_rank = int(_get(m, "q_rank")), \
            int(_get(m, "kv_rank"))
        self.owns_kv = owns_kv
        self.eps = eps
        self.sizes = [self.q_rank, self.kv_rank] if owns_kv \
            else [self.q_rank]
        self.in_proj = MergedColumnParallelLinear(width, self.sizes,
                                                  params_dtype=dtype)
        self.q_norm = nn.Parameter(torch.ones(self.q_rank, dtype=dtype),
                                   requires_grad=False)
        self.uq = ReplicatedLinear(self.q_rank, H * D, params_dtype=dtype)
        self.attn = LatentAttention(kv_index, H, D, Dv, self.kv_rank,
                                    float(_get(m, "scale")), eps,
                                    owns_kv=owns_kv, params_dtype=dtype)
        self.out_proj = RowParallelLinear(H * Dv, width, params_dtype=dtype)

    def forward(self, h: torch.Tensor, fctx: ForwardContext):
        proj = self.in_proj(h)
        cq = ops.rms_weight_store(proj[:, :self.q_rank], self.q_norm,
                                  self.eps)
        ckv = proj[:, self.q_rank:] if self.owns_kv else None
        return self.out_proj(self.attn(self.uq(cq), ckv, fctx))


class ClampedExperts(nn.Module):
    """Top-k-of-logits routing (fp32 router, softmax over the chosen)
    into clamped-SwiGLU experts, plus an optional shared expert of the
    same form whose result is gated per token. Returns (routed, shared
    or None, gate logits [T, 1] or None); the sum routed + sigmoid(gate)
    * shared is formed where the result joins the residual."""

    def __init__(self, width: int, mlp, engine_config, dtype):
        super().__init__()
        router = _get(mlp, "router")
        expert = _get(mlp, "expert")
        self.num_experts = int(_get(router, "experts"))
        self.top = int(_get(router, "top"))
        self.router = ReplicatedLinear(width, self.num_experts,
                                       params_dtype=dtype)
        self.experts = FusedMoE(
            self.num_experts, self.top, width, int(_get(expert, "ff")),
            renormalize=True, use_ep=engine_config.use_ep,
            params_dtype=dtype, activation="swiglu_clamp",
            fp32_routing_weights=True,
            act_limit=float(_get(expert, "limit")), act_alpha=EXPERT_ALPHA)
        shared = _get(mlp, "shared")
        self.shared_ff = int(_get(shared, "ff")) if shared else 0
        if self.shared_ff:
            self.shared_limit = float(_get(shared, "limit"))
            # gate rows | up rows | the one-row result gate, padded with
            # zero rows to 8 so that the rows of the projection's output
            # stay 16 B aligned for the activation kernel
            self.sizes = [self.shared_ff, self.shared_ff, 8]
            self.shared_in = MergedColumnParallelLinear(
                width, self.sizes, params_dtype=dtype)
            self.shared_in.weight.data.zero_()
            self.shared_down = RowParallelLinear(self.shared_ff, width,
                                                 params_dtype=dtype)
        self._r32 = None

    def forward(self, h: torch.Tensor):
        if self._r32 is None or self._r32.device != h.device:
            self._r32 = self.router.weight.float()
        logits = F.linear(h.float(), self._r32)
        weights, ids = ops.topk_then_softmax(logits, self.top)
        y = self.experts.forward_routed(h, weights, ids)
        if not self.shared_ff:
            return y, None, None
        proj = self.shared_in(h)
        act = ops.clamp_swiglu(proj[:, :2 * self.shared_ff],
                               self.shared_limit, EXPERT_ALPHA)
        return y, self.shared_down(act), \
            proj[:, 2 * self.shared_ff:2 * self.shared_ff + 1]


class GopetarLayer(nn.Module):
    def __init__(self, width: int, layer, eps: float, streams: int,
                 engine_config, dtype, kv_index: int, owns_kv: bool,
                 ssm_layer_id: int):
        super().__init__()
        self.kind = _get(layer, "type")
        m = _get(layer, "mixer")
        if self.kind == "parallel":
            self.mix = ParallelMixer(width, m, eps, kv_index, ssm_layer_id,
                                     dtype)
        elif self.kind == "latent_attention":
            self.mix = LatentMixer(width, m, eps, kv_index, owns_kv, dtype)
        else:
            raise ValueError(f"unknown mixer type {self.kind!r}")
        self.hc1 = HyperConnection(streams, eps)
        mlp = _get(layer, "mlp")
        if mlp:
            kind = _get(mlp, "kind", "moe")
            if kind != "moe":
                raise ValueError(f"unknown feed-forward kind {kind!r}")
            self.mlp = ClampedExperts(width, mlp, engine_config, dtype)
            self.hc2 = HyperConnection(streams, eps)
        else:
            self.mlp = None
            self.hc2 = None

    def forward(self, xs: torch.Tensor, h: torch.Tensor,
                fctx: ForwardContext, nxt: HyperConnection):
        """xs: fp32 streams (updated in place); h = what hc1 read.
        Returns what ``nxt`` reads from the updated streams."""
        y = self.mix(h, fctx)
        if self.mlp is None:
            return self.hc1.write(xs, y, nxt)
        h = self.hc1.write(xs, y, self.hc2)
        y, shared, gate = self.mlp(h)
        return self.hc2.write(xs, y, nxt, shared, gate)


class GopetarForCausalLM(nn.Module):
    # the ragged state kernel reads slots / flags from device tensors
    wants_state_tensors = True

    def __init__(self, cfg, engine_config):
        super().__init__()
        from gllm_amd.parallel import get_pp_size, get_tp_size
        assert get_tp_size() == 1 and get_pp_size() == 1, \
            "Gopetar serves on one GPU per replica (tp = pp = 1)"
        self.cfg = cfg
        dtype = engine_config.torch_dtype()
        self.dtype = dtype
        layers = list(cfg.layers)
        width = int(cfg.width)
        vocab = int(cfg.vocab)
        eps = float(_get(cfg.norm, "eps"))
        self.streams = int(getattr(cfg, "streams", 1) or 1)
        self.embed_scale = float(
            _get(getattr(cfg, "embedding", None), "scale", 1.0))
        # names the rest of the framework reads off a model config
        cfg.vocab_size = vocab
        cfg.hidden_size = width
        cfg.num_hidden_layers = len(layers)
        self.layer_start, self.layer_end = 0, len(layers)
        self.is_first_stage = self.is_last_stage = True
        self.embed = VocabParallelEmbedding(vocab, width, params_dtype=dtype)
        mods: List[GopetarLayer] = []
        kv_index_of = {}
        kv_shapes: List[Tuple[int, int, int]] = []
        ssm_specs: List[SSMLayerSpec] = []
        for i, layer in enumerate(layers):
            kind = _get(layer, "type")
            m = _get(layer, "mixer")
            owns, ssm_id = True, -1
            if kind == "parallel":
                left = _get(m, "left")
                kv = len(kv_shapes)
                kv_shapes.append((int(_get(left, "kv_heads")),
                                  int(_get(left, "dim")),
                                  int(_get(left, "vdim"))))
                ssm_id = len(ssm_specs)
            elif kind == "latent_attention":
                src = _get(m, "kv_from")
                if src is None:
                    kv = kv_index_of[i] = len(kv_shapes)
                    # one latent row per token is key and value at once
                    kv_shapes.append((1, int(_get(m, "kv_rank")), 0))
                else:
                    if int(src) not in kv_index_of:
                        raise ValueError(
                            f"layer {i}: kv_from {src} is not an earlier "
                            "latent-attention layer with a latent of its "
                            "own")
                    kv, owns = kv_index_of[int(src)], False
                    if kv_shapes[kv][1] != int(_get(m, "kv_rank")):
                        raise ValueError(
                            f"layer {i}: kv_rank differs from layer {src}")
            else:
                raise ValueError(f"unknown mixer type {kind!r}")
            lay = GopetarLayer(width, layer, eps, self.streams,
                               engine_config, dtype, kv, owns, ssm_id)
            if kind == "parallel":
                ssm_specs.append(lay.mix.gru.spec())
            mods.append(lay)
        self.layers = nn.ModuleList(mods)
        self.kv_layer_shapes = kv_shapes
        self.num_kv_layers = len(kv_shapes)
        self.ssm_spec = None
        if ssm_specs:
            s0 = ssm_specs[0]
            self.ssm_spec = SSMSpec(len(ssm_specs), s0.conv_dim,
                                    s0.conv_kernel, s0.num_v_heads,
                                    s0.head_k_dim, s0.head_v_dim,
                                    layers=ssm_specs)
        # the last read: plain sum of the streams through the final norm
        self.final = sum_reader(self.streams, eps)
        self.lm_head = ParallelLMHead(vocab, width, params_dtype=dtype)
        # hipGraph decode buckets need a sync-free forward: bf16 with
        # every MoE on the grouped GEMM (8-aligned width and ff); fp32
        # and odd expert shapes take the host segment loop
        self.supports_graph = dtype == torch.bfloat16 and all(
            lay.mlp is None or (width % 8 == 0 and
                                lay.mlp.experts.intermediate_per_rank % 8
                                == 0)
            for lay in mods)
        # called as layer_probe(layer index, summed stream) after a layer
        self.layer_probe = None

    @property
    def num_local_layers(self):
        return len(self.layers)

    def forward(self, input_ids, positions, fctx, hidden_states=None,
                residual=None):
        x0 = self.embed(input_ids).float() * self.embed_scale
        xs = x0.unsqueeze(0).repeat(self.streams, 1, 1)
        first = self.layers[0].hc1 if len(self.layers) else self.final
        h = first.read(xs, self.dtype)
        for i, layer in enumerate(self.layers):
            nxt = self.layers[i + 1].hc1 if i + 1 < len(self.layers) \
                else self.final
            h = layer(xs, h, fctx, nxt)
            if self.layer_probe is not None:
                self.layer_probe(i, xs.sum(0))
        return h, None

    def compute_logits(self, hidden_states, fctx):
        rows = hidden_states
        if fctx.logits_indices is not None:
            rows = hidden_states.index_select(0, fctx.logits_indices)
        return self.lm_head(rows)

    # ------------------------------------------------------------------
    def load_weights(self, weights: Iterable[Tuple[str, torch.Tensor]]):
        """Checkpoint names: ``embed``, ``head``, ``final.norm`` and per
        layer ``l<i>.norm{1,2}``, ``l<i>.hc{1,2}.{in,out,mix}``,
        ``l<i>.mix.left.{q,k,v}[.b]``, ``.left.{sink,o}``,
        ``l<i>.mix.right.{z,x}[.b]``, ``.right.{g,o}`` (parallel) or
        ``l<i>.mix.{dq,dq.norm,uq,dkv,dkv.norm,uk,uv,o}`` (latent) and
        ``l<i>.mlp.{router, e<j>.{gate,up,down},
        shared.{gate,up,down,sg}}``."""
        seen = set()
        for name, w in weights:
            if self._load_one(name, w):
                seen.add(name)
            elif w.is_floating_point():
                raise KeyError(f"unexpected tensor {name!r}")
        return seen

    @staticmethod
    def _copy(param, w):
        assert tuple(param.shape) == tuple(w.shape), \
            (tuple(param.shape), tuple(w.shape))
        param.data.copy_(w.to(param.dtype))

    def _load_one(self, name: str, w: torch.Tensor) -> bool:
        if name == "embed":
            self.embed.weight.weight_loader(self.embed.weight, w)
            return True
        if name == "head":
            self.lm_head.weight.weight_loader(self.lm_head.weight, w)
            return True
        if name == "final.norm":
            self.final.norm.load(w)
            return True
        parts = name.split(".")
        if not (parts[0].startswith("l") and parts[0][1:].isdigit()):
            return False
        layer = self.layers[int(parts[0][1:])]
        rest = parts[1:]
        if rest in (["norm1"], ["norm2"]):
            hc = layer.hc1 if rest[0] == "norm1" else layer.hc2
            hc.norm.load(w)
            return True
        if rest[0] in ("hc1", "hc2") and len(rest) == 2:
            hc = getattr(layer, rest[0])
            p = {"in": hc.in_w, "out": hc.out_w, "mix": hc.mix}.get(rest[1])
            if p is None:
                return False
            self._copy(p, w)
            return True
        if rest[0] == "mlp":
            return self._load_mlp(layer.mlp, rest[1:], w)
        if rest[0] != "mix":
            return False
        if isinstance(layer.mix, ParallelMixer):
            return self._load_parallel(layer.mix, rest[1:], w)
        return self._load_latent(layer.mix, rest[1:], w)

    def _load_parallel(self, mix: ParallelMixer, sub: List[str], w) -> bool:
        if len(sub) < 2:
            return False
        shard = mix.SHARDS.get((sub[0], sub[1]))
        if shard is not None and sub[2:] in ([], ["b"]):
            if sub[2:] == ["b"] and sub[1] == "g":
                return False
            p = mix.in_proj.bias if sub[2:] == ["b"] else mix.in_proj.weight
            p.weight_loader(p, w, shard)
            return True
        if sub == ["left", "sink"]:
            self._copy(mix.attn.sinks, w)
            return True
        if sub == ["left", "o"]:
            self._copy(mix.out_proj.weight.data[:, :mix.heads_out], w)
            return True
        if sub == ["right", "o"]:
            self._copy(mix.out_proj.weight.data[:, mix.heads_out:], w)
            return True
        return False

    def _load_latent(self, mix: LatentMixer, sub: List[str], w) -> bool:
        at = mix.attn
        if sub == ["dq"]:
            p = mix.in_proj.weight
            p.weight_loader(p, w, 0)
        elif sub == ["dkv"] and mix.owns_kv:
            p = mix.in_proj.weight
            p.weight_loader(p, w, 1)
        elif sub == ["dq", "norm"]:
            self._copy(mix.q_norm, w)
        elif sub == ["dkv", "norm"] and mix.owns_kv:
            self._copy(at.kv_norm, w)
        elif sub == ["uq"]:
            self._copy(mix.uq.weight, w)
        elif sub == ["uk"]:
            self._copy(at.w_uk.data.view(-1, at.rank), w)
        elif sub == ["uv"]:
            self._copy(at.w_uv.data.view(-1, at.rank), w)
        elif sub == ["o"]:
            self._copy(mix.out_proj.weight, w)
        else:
            return False
        return True

    def _load_mlp(self, mlp: ClampedExperts, sub: List[str], w) -> bool:
        if mlp is None:
            return False
        if sub == ["router"]:
            self._copy(mlp.router.weight, w)
            return True
        if len(sub) == 2 and sub[0] == "shared" and mlp.shared_ff:
            if sub[1] == "down":
                self._copy(mlp.shared_down.weight, w)
                return True
            if sub[1] == "sg":
                self._copy(mlp.shared_in.weight.data[
                    2 * mlp.shared_ff:2 * mlp.shared_ff + 1], w)
                return True
            shard = {"gate": 0, "up": 1}.get(sub[1])
            if shard is None:
                return False
            p = mlp.shared_in.weight
            p.weight_loader(p, w, shard)
            return True
        if len(sub) == 2 and sub[0].startswith("e") and sub[0][1:].isdigit():
            e = int(sub[0][1:])
            ex = mlp.experts
            if sub[1] == "gate":
                ex.w13_weight.weight_loader(ex.w13_weight, w, e, 0)
            elif sub[1] == "up":
                ex.w13_weight.weight_loader(ex.w13_weight, w, e, 1)
            elif sub[1] == "down":
                ex.w2_weight.weight_loader(ex.w2_weight, w, e)
            else:
                return False
            return True
        return False
