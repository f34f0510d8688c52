"""Sofunex: a config-driven looped decoder whose mixer runs windowed
attention and a generalized delta rule side by side.

``config.layers`` describes every layer on its own (mixer sizes and the
feed-forward: dense, mixture of experts, or none), so sizes may differ
from layer to layer. ``config.loop`` = {start, stop, times} runs layers
start..stop-1 ``times`` times in a row with the same weights; every run
of a layer owns a KV cache and a state-pool entry of its own, and pass
t opens with x += loop.step[t].

* stream: fp32, embed[token] * embedding.scale; every sublayer is
  x += residual_mult * RMSnorm_post(f(RMSnorm_pre(x))) with plain
  weights
* token shift: the mixer reads h_t + (h_(t-1) - h_t) * shift, the
  previous token's normed row being part of the sequence's state
* mixer ``parallel``: left_scale * left + right_scale * right on the
  same input —
  left: GQA with biased q/k/v/o, a short causal convolution over time
  on every q/k/v channel (no activation), ONE RMS norm over the whole
  q row (and k row) with row-sized weights, rotate-half rotary on the
  first ``rot.dims`` dims with linear position scaling, unit-RMS value
  heads, a sliding window and an ordinary softmax;
  right: delta rule with per-channel decay (a low-rank tanh branch) and
  per-channel removal rate on the unit key, fp32 state per sequence,
  read out through a per-head RMS norm with row-sized weights and a
  sigmoid gate
* feed-forward: dense gelu_tanh GLU, or sigmoid-router MoE of SiLU-GLU
  experts (selection on score + correction within the best groups,
  weights = chosen scores over their sum, times router.scale) plus an
  always-on shared expert

Framework mapping: ONE merged input projection per mixer (q | k | v |
r | k | v | g | a | w1, biases on the merged bias) and ONE output GEMM
over [attention heads | gated read-out] (layers/linear.py),
StreamRMSNorm.add_into = one launch per sublayer boundary
(layers/layernorm.py), TokenShift + GeneralDeltaRule over the state
pool (layers/recurrent.py, core/ssm.py), WindowAttention with
``norm_span`` / ``value_unit_norm`` + HalfRotary (layers/attention.py,
layers/rotary.py), FusedMoE (layers/moe/layer.py), the paged KV pool
with one entry per layer RUN (core/kv_cache.py). Prompt portions and
decode tokens of a mixed batch go through the same ragged kernels.
"""

import math
from typing import Iterable, List, Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from gllm_amd import ops
from gllm_amd.core.ssm import SSMLayerSpec, SSMSpec
from gllm_amd.layers.attention import WindowAttention
from gllm_amd.layers.embedding import ParallelLMHead, VocabParallelEmbedding
from gllm_amd.layers.layernorm import StreamRMSNorm
from gllm_amd.layers.linear import (MergedColumnParallelLinear,
                                    ReplicatedLinear, RowParallelLinear)
from gllm_amd.layers.moe.layer import FusedMoE
from gllm_amd.layers.recurrent import (GeneralDeltaRule, TokenShift,
                                       state_rows)
from gllm_amd.layers.rotary import HalfRotary
from gllm_amd.runtime.forward_context import ForwardContext

# the decay of a key channel is exp(-DECAY_SCALE * sigmoid(.)): it stays
# inside (exp(-DECAY_SCALE), 1)
DECAY_SCALE = math.exp(-0.5)


def _get(d, key, default=None):
    """config.json sub-objects arrive as dicts (or namespaces)."""
    if d is None:
        return default
    if isinstance(d, dict):
        return d.get(key, default)
    return getattr(d, key, default)


class ConvAttentionDeltaMixer(nn.Module):
    """Convolved windowed attention beside a generalized delta rule:
    one input GEMM, one output GEMM over [heads | read-out]."""

    # column blocks of the merged projection, in order
    SHARDS = {("left", "q"): 0, ("left", "k"): 1, ("left", "v"): 2,
              ("right", "r"): 3, ("right", "k"): 4, ("right", "v"): 5,
              ("right", "g"): 6, ("right", "a"): 7, ("right", "w1"): 8}

    def __init__(self, width: int, m, eps: float, dtype):
        super().__init__()
        left, right = _get(m, "left"), _get(m, "right")
        H, D = int(_get(left, "heads")), int(_get(left, "dim"))
        G = int(_get(left, "kv_heads", H) or H)
        Dv = int(_get(left, "vdim", D) or D)
        Hr, Dr = int(_get(right, "heads")), int(_get(right, "dim"))
        self.R = R = Hr * Dr
        self.kv_shape = (G, D, Dv)
        self.left_scale = float(_get(m, "left_scale", 1.0))
        self.right_scale = float(_get(m, "right_scale", 1.0))
        # the output GEMM sees [heads | c * read-out] and the norm that
        # follows multiplies by left_scale in fp32 (c = right / left):
        # no weight, bias or activation is rounded a second time
        self.y_scale = self.left_scale if self.left_scale != 0.0 else 1.0
        self.left_mul = self.left_scale / self.y_scale
        self.right_mul = self.right_scale / self.y_scale
        # taps of the short convolution; 0 = the layer has none (a
        # one-tap convolution is a per-channel factor and keeps its
        # weights)
        self.taps = int(_get(left, "conv", 0) or 0)
        self.attn_sizes = [H * D, G * D, G * Dv]
        self.conv_dim = sum(self.attn_sizes)
        # the decay's low-rank width comes with the checkpoint; the
        # projection is sized when its tensor arrives
        self.rank = int(_get(right, "decay_rank", 0) or 0)
        self.width = width
        self.dtype = dtype
        self.in_proj = None
        self.w2 = None
        self._pending = []      # tensors that arrived before w1
        if self.rank:
            self._size(self.rank)
        if self.taps >= 1:
            self.conv_weight = nn.Parameter(
                torch.zeros(self.conv_dim, self.taps, dtype=dtype),
                requires_grad=False)
            self.conv_weight.data[:, -1] = 1.0
        self.heads_out = H * Dv
        self.out_proj = RowParallelLinear(H * Dv + R, width, bias=True,
                                          params_dtype=dtype)
        self.out_proj.bias.data.zero_()
        rot = _get(left, "rot")
        rotary = None
        if rot and int(_get(rot, "dims", 0) or 0) > 0:
            rotary = HalfRotary(int(_get(rot, "dims")),
                                float(_get(rot, "base")),
                                _get(rot, "scaling"))
        mask = _get(left, "mask")
        self.attn = WindowAttention(
            -1, H, G, D, Dv, float(_get(left, "scale", D ** -0.5)), eps,
            window=int(_get(mask, "size", 0) or 0), sink=False,
            rotary=rotary, params_dtype=dtype, qk_norm=True,
            norm_span=True, value_unit_norm=True)
        self.delta = GeneralDeltaRule(Hr, Dr, Dr, eps, -1, DECAY_SCALE,
                                      params_dtype=dtype)

    def _size(self, rank: int):
        self.rank = rank
        R = self.R
        self.sizes = self.attn_sizes + [R, R, R, R, R, rank]
        dev = self.out_proj.weight.device if hasattr(self, "out_proj") \
            else None
        self.in_proj = MergedColumnParallelLinear(
            self.width, self.sizes, bias=True, params_dtype=self.dtype)
        self.in_proj.bias.data.zero_()
        self.w2 = ReplicatedLinear(rank, R, params_dtype=self.dtype)
        if dev is not None:
            self.in_proj.to(dev)
            self.w2.to(dev)

    def spec(self, width: int) -> SSMLayerSpec:
        return self.delta.spec(self.conv_dim if self.taps >= 1 else 0,
                               max(self.taps, 1), shift_dim=width)

    def forward(self, h: torch.Tensor, fctx: ForwardContext, kv_index: int,
                ssm_id: int):
        """Returns (y, y_scale): the mixer's result is y_scale * y."""
        T = h.shape[0]
        proj = self.in_proj(h)
        qkv = proj[:, :self.conv_dim]
        if self.taps >= 1 and not fctx.is_profile_run \
                and fctx.ssm_pool is not None:
            slots, init = state_rows(fctx, T, h.device)
            qkv = ops.causal_conv_silu(
                qkv, self.conv_weight, fctx.ssm_pool.conv_state[ssm_id],
                slots, init, fctx.query_start_loc, activation=False,
                max_query_len=fctx.max_query_len)
        q, k, v = qkv.split(self.attn_sizes, dim=-1)
        R, c0 = self.R, self.conv_dim
        r, k2, v2, g, a = (proj[:, c0 + i * R:c0 + (i + 1) * R]
                           for i in range(5))
        w_logit = self.w2(ops.tanh_rows(proj[:, c0 + 5 * R:]))
        both = torch.empty(T, self.heads_out + R, dtype=h.dtype,
                           device=h.device)
        self.attn(q, k, v, None, fctx, out=both[:, :self.heads_out],
                  out_scale=self.left_mul, layer_idx=kv_index)
        self.delta(r, k2, v2, w_logit, a, g, fctx,
                   out=both[:, self.heads_out:], scale=self.right_mul,
                   ssm_layer_id=ssm_id)
        return self.out_proj(both), self.y_scale


class DenseGLU(nn.Module):
    """gate | up in one projection -> gelu_tanh(gate) * up -> down."""

    def __init__(self, width: int, mlp, dtype):
        super().__init__()
        ff = int(_get(mlp, "ff"))
        self.in_proj = MergedColumnParallelLinear(width, [ff, ff],
                                                  params_dtype=dtype)
        self.down = RowParallelLinear(ff, width, params_dtype=dtype)

    def forward(self, h: torch.Tensor):
        return self.down(ops.gated_act_mul(self.in_proj(h), "gelu_tanh")), None


class GroupRoutedExperts(nn.Module):
    """fp32 sigmoid router with a selection-only correction and group
    limits -> SiLU-GLU experts, plus an optional always-on shared
    expert. Returns (routed, shared or None); the sum is formed where
    the result joins the residual."""

    def __init__(self, width: int, mlp, engine_config, dtype):
        super().__init__()
        router = _get(mlp, "router")
        self.num_experts = int(_get(router, "experts"))
        self.top = int(_get(router, "top"))
        groups = _get(router, "groups")
        self.n_group = int(_get(groups, "count", 1) or 1)
        self.keep = int(_get(groups, "keep", self.n_group) or self.n_group)
        if self.num_experts % self.n_group:
            raise ValueError("router.groups.count must divide the experts")
        self.scale = float(_get(router, "scale", 1.0))
        self.router = ReplicatedLinear(width, self.num_experts,
                                       params_dtype=dtype)
        self.correction = nn.Parameter(
            torch.zeros(self.num_experts, dtype=torch.float32),
            requires_grad=False)
        self.experts = FusedMoE(
            self.num_experts, self.top, width,
            int(_get(_get(mlp, "expert"), "ff")), renormalize=False,
            use_ep=engine_config.use_ep, params_dtype=dtype,
            fp32_routing_weights=True)
        shared = _get(mlp, "shared")
        self.shared_ff = int(_get(shared, "ff")) if shared else 0
        if self.shared_ff:
            self.shared_in = MergedColumnParallelLinear(
                width, [self.shared_ff, self.shared_ff], params_dtype=dtype)
            self.shared_down = RowParallelLinear(self.shared_ff, width,
                                                 params_dtype=dtype)
        self._r32 = None

    def forward(self, h: torch.Tensor):
        if self._r32 is None or self._r32.device != h.device:
            self._r32 = self.router.weight.float()
        logits = F.linear(h.float(), self._r32)
        weights, ids = ops.sigmoid_group_topk(
            logits, self.correction, self.top, self.n_group, self.keep,
            self.scale)
        y = self.experts.forward_routed(h, weights, ids)
        if not self.shared_ff:
            return y, None
        return y, self.shared_down(ops.gated_act_mul(self.shared_in(h), "silu"))


class SofunexLayer(nn.Module):
    def __init__(self, width: int, layer, eps: float, mult: float,
                 engine_config, dtype):
        super().__init__()
        kind = _get(layer, "type")
        if kind != "parallel":
            raise ValueError(f"unknown mixer type {kind!r}")
        self.mult = mult
        self.mix = ConvAttentionDeltaMixer(width, _get(layer, "mixer"), eps,
                                           dtype)
        self.shift = TokenShift(width, -1, params_dtype=dtype)
        self.norm1 = StreamRMSNorm(width, eps, dtype)
        self.norm1b = StreamRMSNorm(width, eps, dtype)
        mlp = _get(layer, "mlp")
        if mlp:
            kind = _get(mlp, "kind")
            if kind == "dense":
                self.mlp = DenseGLU(width, mlp, dtype)
            elif kind == "moe":
                self.mlp = GroupRoutedExperts(width, mlp, engine_config,
                                              dtype)
            else:
                raise ValueError(f"unknown feed-forward kind {kind!r}")
            self.norm2 = StreamRMSNorm(width, eps, dtype)
            self.norm2b = StreamRMSNorm(width, eps, dtype)
        else:
            self.mlp = None

    def forward(self, x: torch.Tensor, h: torch.Tensor,
                fctx: ForwardContext, nxt: Optional[StreamRMSNorm],
                run: int, add: Optional[torch.Tensor] = None):
        """x: fp32 stream (updated in place); h = norm1(x). ``run``
        indexes this run's KV cache and state-pool entry. Returns
        ``nxt`` applied to the updated x (+ ``add``), None without
        ``nxt``."""
        h = self.shift(h, fctx, run)
        y, ys = self.mix(h, fctx, run, run)
        if self.mlp is None:
            return self.norm1b.add_into(x, y, nxt, self.mult, ys, add=add)
        h = self.norm1b.add_into(x, y, self.norm2, self.mult, ys)
        y, y2 = self.mlp(h)
        return self.norm2b.add_into(x, y, nxt, self.mult, 1.0, y2, add)


class SofunexForCausalLM(nn.Module):
    # the ragged state kernels read slots / flags from device tensors
    wants_state_tensors = True

    def __init__(self, cfg, engine_config):
        super().__init__()
        from gllm_amd.parallel import get_pp_size, get_tp_size
        assert get_tp_size() == 1 and get_pp_size() == 1, \
            "Sofunex serves on one GPU per replica (tp = pp = 1)"
        self.cfg = cfg
        dtype = engine_config.torch_dtype()
        self.dtype = dtype
        layers = list(cfg.layers)
        width = int(cfg.width)
        vocab = int(cfg.vocab)
        eps = float(_get(cfg.norm, "eps"))
        mult = float(getattr(cfg, "residual_mult", 1.0))
        self.embed_scale = float(
            _get(getattr(cfg, "embedding", None), "scale", 1.0))
        # names the rest of the framework reads off a model config
        cfg.vocab_size = vocab
        cfg.hidden_size = width
        cfg.num_hidden_layers = len(layers)
        self.layer_start, self.layer_end = 0, len(layers)
        self.is_first_stage = self.is_last_stage = True
        self.embed = VocabParallelEmbedding(vocab, width, params_dtype=dtype)
        self.layers = nn.ModuleList(
            SofunexLayer(width, layer, eps, mult, engine_config, dtype)
            for layer in layers)
        # the order layers run in: (layer, pass it opens or None)
        loop = getattr(cfg, "loop", None)
        n = len(layers)
        if loop:
            a, b = int(_get(loop, "start")), int(_get(loop, "stop"))
            times = int(_get(loop, "times"))
            if not 0 <= a <= b <= n or times < 1:
                raise ValueError(f"bad loop {loop!r} for {n} layers")
            order = [(i, None) for i in range(a)]
            for t in range(times):
                order += [(i, t if i == a else None) for i in range(a, b)]
            order += [(i, None) for i in range(b, n)]
            # fp32: it joins the fp32 stream as it is
            self.loop_step = nn.Parameter(
                torch.zeros(times, width, dtype=torch.float32),
                requires_grad=False)
        else:
            order = [(i, None) for i in range(n)]
            self.loop_step = None
        self.runs: List[Tuple[int, Optional[int]]] = order
        self.kv_layer_shapes = [self.layers[li].mix.kv_shape
                                for li, _ in order]
        self.num_kv_layers = len(self.kv_layer_shapes)
        self.width = width
        self.ssm_spec = None
        self._build_ssm_spec()
        self.final_norm = StreamRMSNorm(width, eps, dtype)
        self.lm_head = ParallelLMHead(vocab, width, params_dtype=dtype)
        # hipGraph decode buckets need a sync-free forward: bf16 with
        # every MoE on the grouped GEMM (8-aligned width and ff)
        self.supports_graph = dtype == torch.bfloat16 and all(
            not isinstance(lay.mlp, GroupRoutedExperts) or
            (width % 8 == 0 and
             lay.mlp.experts.intermediate_per_rank % 8 == 0)
            for lay in self.layers)
        # called as layer_probe(run index, x) after every layer run
        self.layer_probe = None

    def _build_ssm_spec(self):
        specs = [self.layers[li].mix.spec(self.width) for li, _ in self.runs]
        if specs:
            s0 = specs[0]
            self.ssm_spec = SSMSpec(len(specs), s0.conv_dim, s0.conv_kernel,
                                    s0.num_v_heads, s0.head_k_dim,
                                    s0.head_v_dim, layers=specs)

    @property
    def num_local_layers(self):
        return len(self.layers)

    def _step(self, opens: Optional[int]):
        return None if opens is None else self.loop_step[opens]

    def forward(self, input_ids, positions, fctx, hidden_states=None,
                residual=None):
        x = self.embed(input_ids).float() * self.embed_scale
        h = None
        last = len(self.runs) - 1
        probing = self.layer_probe is not None
        for r, (li, opens) in enumerate(self.runs):
            layer = self.layers[li]
            if h is None:
                h = layer.norm1(x, add=self._step(opens))
            if probing:
                nxt, add = None, None
            elif r == last:
                nxt, add = self.final_norm, None
            else:
                nli, nopens = self.runs[r + 1]
                nxt, add = self.layers[nli].norm1, self._step(nopens)
            h = layer(x, h, fctx, nxt, r, add)
            if probing:
                self.layer_probe(r, x)
        if h is None:
            h = self.final_norm(x)
        return h, None

    def compute_logits(self, hidden_states, fctx):
        rows = hidden_states
        if fctx.logits_indices is not None:
            rows = hidden_states.index_select(0, fctx.logits_indices)
        return self.lm_head(rows)

    # ------------------------------------------------------------------
    def load_weights(self, weights: Iterable[Tuple[str, torch.Tensor]]):
        """Checkpoint names: ``embed``, ``head``, ``final.norm``,
        ``loop.step`` and per layer ``l<i>.norm{1,1b,2,2b}``,
        ``l<i>.shift``, ``l<i>.mix.left.{q,k,v}[.b|.conv|.norm]``,
        ``.left.o[.b]``, ``l<i>.mix.right.{r,k,v,g,a,a.b,w1,w2,w0,norm,
        o}`` and ``l<i>.mlp.{gate,up,down}`` (dense) or ``l<i>.mlp.
        {router, correction, e<j>.{gate,up,down}, shared.{gate,up,
        down}}``."""
        seen = set()
        for name, w in weights:
            if self._load_one(name, w):
                seen.add(name)
            elif w.is_floating_point():
                raise KeyError(f"unexpected tensor {name!r}")
        for i, layer in enumerate(self.layers):
            if layer.mix.in_proj is None:
                raise KeyError(f"l{i}.mix.right.w1 is missing")
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
            self._copy(self.final_norm.weight, w)
            return True
        if name == "loop.step" and self.loop_step is not None:
            self._copy(self.loop_step, w)
            return True
        parts = name.split(".")
        if not (parts[0].startswith("l") and parts[0][1:].isdigit()):
            return False
        layer = self.layers[int(parts[0][1:])]
        rest = parts[1:]
        if len(rest) == 1 and rest[0] in ("norm1", "norm1b", "norm2",
                                          "norm2b"):
            norm = getattr(layer, rest[0], None)
            if norm is None:
                return False
            self._copy(norm.weight, w)
            return True
        if rest == ["shift"]:
            self._copy(layer.shift.mu, w)
            return True
        if rest[0] == "mlp":
            return self._load_mlp(layer.mlp, rest[1:], w)
        if rest[0] != "mix" or len(rest) < 3:
            return False
        return self._load_mix(layer.mix, rest[1], rest[2:], w)

    def _load_mix(self, mix: ConvAttentionDeltaMixer, side: str,
                  sub: List[str], w) -> bool:
        if mix.in_proj is None:
            # the merged projection is sized by w1's row count: hold
            # the mixer's other tensors until it has arrived
            if (side, sub) != ("right", ["w1"]):
                mix._pending.append((side, sub, w))
                return True
            mix._size(int(w.shape[0]))
            pending, mix._pending = mix._pending, []
            for ps, pn, pw in pending:
                if not self._load_mix(mix, ps, pn, pw) \
                        and pw.is_floating_point():
                    raise KeyError(f"unexpected tensor {ps}.{'.'.join(pn)}")
        shard = mix.SHARDS.get((side, sub[0]))
        at, dl = mix.attn, mix.delta
        if shard is not None and sub[1:] == []:
            p = mix.in_proj.weight
            p.weight_loader(p, w, shard)
            return True
        if shard is not None and sub[1:] == ["b"] and (
                side == "left" or sub[0] == "a"):
            p = mix.in_proj.bias
            p.weight_loader(p, w, shard)
            return True
        if side == "left":
            if sub[1:] == ["conv"] and sub[0] in ("q", "k", "v") \
                    and mix.taps >= 1:
                off = sum(mix.attn_sizes[:shard])
                self._copy(mix.conv_weight.data.narrow(0, off, w.shape[0]),
                           w)
                return True
            if sub == ["q", "norm"]:
                self._copy(at.q_norm, w)
                return True
            if sub == ["k", "norm"]:
                self._copy(at.k_norm, w)
                return True
            if sub == ["o"]:
                self._copy(mix.out_proj.weight.data[:, :mix.heads_out], w)
                return True
            if sub == ["o", "b"]:
                self._copy(mix.out_proj.bias, w)
                if mix.left_scale == 0.0:
                    mix.out_proj.bias.data.zero_()
                return True
            return False
        if side != "right":
            return False
        if sub == ["w2"]:
            self._copy(mix.w2.weight, w)
        elif sub == ["w0"]:
            self._copy(dl.w0, w)
        elif sub == ["norm"]:
            self._copy(dl.norm_weight, w)
        elif sub == ["o"]:
            self._copy(mix.out_proj.weight.data[:, mix.heads_out:], w)
        else:
            return False
        return True

    @staticmethod
    def _glu_shard(proj, down, which: str, w) -> bool:
        if which == "down":
            p = down.weight
            p.weight_loader(p, w)
            return True
        shard = {"gate": 0, "up": 1}.get(which)
        if shard is None:
            return False
        p = proj.weight
        p.weight_loader(p, w, shard)
        return True

    def _load_mlp(self, mlp, sub: List[str], w) -> bool:
        if mlp is None:
            return False
        if isinstance(mlp, DenseGLU):
            return len(sub) == 1 and self._glu_shard(mlp.in_proj, mlp.down,
                                                     sub[0], w)
        if sub == ["router"]:
            self._copy(mlp.router.weight, w)
            return True
        if sub == ["correction"]:
            self._copy(mlp.correction, w)
            return True
        if len(sub) == 2 and sub[0] == "shared" and mlp.shared_ff:
            return self._glu_shard(mlp.shared_in, mlp.shared_down, sub[1],
                                   w)
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
