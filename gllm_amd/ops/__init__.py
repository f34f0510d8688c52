"""Custom-op facade — the single switch point between backends.

Mirrors the role of the reference's ``_custom_ops.py`` ("single point
where we can swap backends", _custom_ops.py:1-10): every layer calls
through here. Dispatch rule:

* CUDA (= HIP/ROCm) tensors -> the in-tree gfx950 extension
  ``gllm_amd._kernels``. If the extension is missing on a GPU box this
  RAISES — no silent eager fallback (a GPU run must exercise the native
  kernels).
* CPU tensors -> the PyTorch reference implementations (ops.torch_ref),
  which double as the numerics oracle for the HIP kernels.
"""

from typing import Optional

import torch

from gllm_amd.ops import torch_ref

_K = None
_K_ERR: Optional[str] = None


def _load_kernels():
    global _K, _K_ERR
    if _K is not None or _K_ERR is not None:
        return _K
    try:
        from gllm_amd import _kernels  # built in-tree by setup.py
        _K = _kernels
    except ImportError as e:  # pragma: no cover
        _K_ERR = str(e)
    return _K


_KS = None
_KS_ERR: Optional[str] = None


def _load_seq_kernels():
    """The dtype-generic sequence-mixer module (setup.py SEQ_SOURCES):
    built on its own so a model that needs only these kernels serves
    from a checkout where the full extension was never compiled."""
    global _KS, _KS_ERR
    if _KS is not None or _KS_ERR is not None:
        return _KS
    try:
        from gllm_amd import _kernels_seq
        _KS = _kernels_seq
    except ImportError as e:  # pragma: no cover
        _KS_ERR = str(e)
    return _KS


class _SeqBacked:
    """Stand-in for the full extension when only the sequence-mixer
    module is built: serves the entry points both modules define (MoE
    grouped GEMM, gated activations) and fails loudly on the rest."""

    def __init__(self, mod):
        self._mod = mod

    def __getattr__(self, name):
        try:
            return getattr(self._mod, name)
        except AttributeError:
            raise RuntimeError(
                f"kernel {name!r} lives in gllm_amd._kernels, which is "
                f"not built (import error: {_K_ERR}); run `python "
                "setup.py build_ext --inplace`") from None


def _gpu_kernels():
    k = _load_kernels()
    if k is None:
        ks = _load_seq_kernels()
        if ks is not None:
            return _SeqBacked(ks)
        raise RuntimeError(
            "gllm_amd._kernels HIP extension not built but a CUDA tensor "
            "was passed — build with `python setup.py build_ext --inplace` "
            f"(PYTORCH_ROCM_ARCH=gfx950). Import error: {_K_ERR}")
    return k


def _seq_kernels():
    k = _load_seq_kernels()
    if k is None:
        raise RuntimeError(
            "gllm_amd._kernels_seq HIP extension not built but a CUDA "
            "tensor was passed — build with `GLLM_EXT=seq python setup.py "
            f"build_ext --inplace`. Import error: {_KS_ERR}")
    return k


def has_kernels() -> bool:
    return _load_kernels() is not None


def has_moe_kernels() -> bool:
    """The bf16 grouped MoE GEMM ships in both extension modules."""
    return _load_kernels() is not None or _load_seq_kernels() is not None


# --------------------------------------------------------------- norm
def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    if x.is_cuda:
        out = torch.empty_like(x)
        _gpu_kernels().rmsnorm(out, x, weight, eps)
        return out
    return torch_ref.rmsnorm(x, weight, eps)


def fused_add_rmsnorm(x: torch.Tensor, residual: torch.Tensor,
                      weight: torch.Tensor, eps: float):
    if x.is_cuda:
        _gpu_kernels().fused_add_rmsnorm(x, residual, weight, eps)
        return x, residual
    return torch_ref.fused_add_rmsnorm(x, residual, weight, eps)


# --------------------------------------------------------------- activation
def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    if x.is_cuda:
        d = x.shape[-1] // 2
        out = torch.empty(x.shape[:-1] + (d,), dtype=x.dtype, device=x.device)
        _gpu_kernels().silu_and_mul(out, x)
        return out
    return torch_ref.silu_and_mul(x)


def gelu_and_mul(x: torch.Tensor) -> torch.Tensor:
    if x.is_cuda:
        d = x.shape[-1] // 2
        out = torch.empty(x.shape[:-1] + (d,), dtype=x.dtype, device=x.device)
        _gpu_kernels().gelu_and_mul(out, x)
        return out
    return torch_ref.gelu_and_mul(x)


# --------------------------------------------------------------- rope
def rotary_embedding(positions: torch.Tensor, q: torch.Tensor,
                     k: torch.Tensor, head_dim: int,
                     cos_sin_cache: torch.Tensor, is_neox: bool = True):
    if q.is_cuda:
        _gpu_kernels().rotary_embedding(positions, q, k, head_dim,
                                        cos_sin_cache, is_neox)
        return q, k
    return torch_ref.rotary_embedding(positions, q, k, head_dim,
                                      cos_sin_cache, is_neox)


# --------------------------------------------------------------- kv cache
def reshape_and_cache(k: torch.Tensor, v: torch.Tensor,
                      k_cache: torch.Tensor, v_cache: torch.Tensor,
                      slot_mapping: torch.Tensor):
    if k.is_cuda:
        _gpu_kernels().reshape_and_cache(k, v, k_cache, v_cache, slot_mapping)
        return
    torch_ref.reshape_and_cache(k, v, k_cache, v_cache, slot_mapping)


# --------------------------------------------------------------- attention
def paged_attention(q: torch.Tensor, k_cache: torch.Tensor,
                    v_cache: torch.Tensor, block_table: torch.Tensor,
                    seq_lens: torch.Tensor, query_start_loc: torch.Tensor,
                    scale: float, max_query_len: int = 1,
                    out: Optional[torch.Tensor] = None,
                    sliding_window: int = 0) -> torch.Tensor:
    if q.is_cuda:
        kern = _gpu_kernels()
        if out is None:
            out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
        if max_query_len == 1:
            kern.paged_attention_decode(
                out, q, k_cache, v_cache, block_table, seq_lens, scale,
                sliding_window)
        else:
            kern.paged_attention_prefill(
                out, q, k_cache, v_cache, block_table, seq_lens,
                query_start_loc.int(), max_query_len, scale, sliding_window)
        return out
    return torch_ref.paged_attention(q, k_cache, v_cache, block_table,
                                     seq_lens, query_start_loc, scale,
                                     out=out, sliding_window=sliding_window)


# --------------------------------------------------------------- moe
def topk_softmax(gating: torch.Tensor, topk: int, renormalize: bool = True):
    return torch_ref.topk_softmax(gating, topk, renormalize)


def topk_then_softmax(logits: torch.Tensor, topk: int):
    """Top-k over raw router logits, softmax over the chosen only:
    (weights fp32 [T, k] in descending order of logit, ids int32
    [T, k]). fp32 logits of up to 512 experts on the GPU take one
    wave-per-row kernel (ties go to the lower index)."""
    if (logits.is_cuda and logits.dtype == torch.float32
            and logits.dim() == 2 and logits.shape[1] <= 512
            and topk <= min(64, logits.shape[1])):
        logits = logits.contiguous()
        weights = torch.empty(logits.shape[0], topk, dtype=torch.float32,
                              device=logits.device)
        ids = torch.empty(logits.shape[0], topk, dtype=torch.int32,
                          device=logits.device)
        _seq_kernels().topk_softmax_rows(weights, ids, logits)
        return weights, ids
    return torch_ref.topk_then_softmax(logits, topk)


def grouped_topk(scores, topk, n_group, topk_group, renormalize=True,
                 scoring="softmax", e_bias=None):
    # device-resident (a CPU round-trip here would sync every MoE
    # layer of every DeepSeek step)
    return torch_ref.grouped_topk(scores, topk, n_group, topk_group,
                                  renormalize, scoring, e_bias)


def fused_moe(x: torch.Tensor, w13: torch.Tensor, w2: torch.Tensor,
              topk_weights: torch.Tensor, topk_ids: torch.Tensor,
              expert_start: int = 0,
              num_global_experts: Optional[int] = None,
              activation: str = "silu_glu",
              act_args: tuple = ()) -> torch.Tensor:
    """Grouped-GEMM fused MoE on the gfx950 kernels (GPU, bf16).
    ``activation``: "silu_glu" (w13 = gate | up rows), "relu2"
    (ungated experts, w13 = up rows only, act = max(z, 0)^2) or
    "swiglu_clamp" (w13 = gate | up rows, ``act_args`` = (limit,
    alpha): min(g, limit) * sigmoid(alpha g) * (clamp(u) + 1)).

    Reference fused_experts_impl (fused_moe_triton/fused_moe.py:779):
    align -> GEMM1 -> silu_and_mul -> GEMM2 (weighted scatter) -> sum.
    Fully device-resident and hipGraph-safe (no host syncs; grids are
    sized by upper bound and gated on the device-side block count).
    Returns the PARTIAL output for this rank's expert shard (callers
    run their TP/EP all-reduce on top).
    """
    T, K = x.shape
    E_local, two_i, _ = w13.shape
    topk = topk_ids.shape[1]
    n_pairs = T * topk
    # tile heuristic: match block_m to the expected rows per expert so
    # decode doesn't re-stream expert weights per m-block; large dense
    # batches use the wide-BN prefill variant (gemm code 164 = BM 64 x
    # BN 256 — quarters the A-tile re-reads that dominate prefill)
    rpe = n_pairs / max(1, E_local)
    if n_pairs >= 4096:
        align_m, gemm_m = 64, 164
    elif rpe < 12:
        align_m = gemm_m = 16
    elif rpe < 40:
        align_m = gemm_m = 32
    else:
        align_m = gemm_m = 64
    cap = n_pairs + E_local * (align_m - 1) + 1
    max_blocks = (n_pairs + align_m - 1) // align_m + E_local
    dev = x.device
    k = _gpu_kernels()
    ids32 = topk_ids.int().contiguous()
    sorted_ids = torch.empty(cap, dtype=torch.int32, device=dev)
    expert_blocks = torch.empty(max_blocks, dtype=torch.int32, device=dev)
    n_post = torch.empty(1, dtype=torch.int32, device=dev)
    k.moe_align(ids32, E_local, expert_start, align_m, sorted_ids,
                expert_blocks, n_post)
    rows_pad = cap - 1 + align_m  # >= n_post_pad upper bound
    inter1 = torch.empty(rows_pad, two_i, dtype=x.dtype, device=dev)
    k.moe_gemm(inter1, x, w13, sorted_ids, expert_blocks, n_post, None,
               n_pairs, topk, gemm_m, False)
    if activation == "relu2":
        act = relu2(inter1)
    elif activation == "swiglu_clamp":
        act = clamp_swiglu(inter1, *act_args)
    else:
        act = silu_and_mul(inter1)
    # zero-filled: pairs routed to non-local experts (EP shards) or to
    # the DP padding id -1 are dropped by the align kernel and must
    # contribute zeros
    pair_out = x.new_zeros(n_pairs, K)
    k.moe_gemm(pair_out, act, w2, sorted_ids, expert_blocks, n_post,
               topk_weights.float().contiguous(), n_pairs, topk, gemm_m,
               True)
    out = torch.empty(T, K, dtype=x.dtype, device=dev)
    k.moe_sum(out, pair_out, topk)
    return out


# --------------------------------------------------------------- fp8
def per_token_group_quant_fp8(x: torch.Tensor, group: int = 128,
                              ue8m0: bool = False,
                              transposed: bool = False):
    """[T, K] bf16 -> (e4m3 [T, K], fp32 scales [T, K/group]).
    GPU kernel; CPU callers use the torch math in quantization/fp8.py.
    ``transposed=True`` additionally returns scales_t [K/group, T]
    (column-major) — the skinny GEMM stages a k-group's scales as ONE
    contiguous run instead of a strided 64-line gather."""
    assert x.is_cuda and group == 128
    T, K = x.shape
    q = torch.empty(T, K, dtype=torch.float8_e4m3fn, device=x.device)
    scales = torch.empty(T, K // group, dtype=torch.float32,
                         device=x.device)
    st = torch.empty(K // group, T, dtype=torch.float32,
                     device=x.device) if transposed else None
    _gpu_kernels().per_token_group_quant_fp8(
        x.contiguous(), q.view(torch.uint8), scales, st, ue8m0)
    if transposed:
        return q, scales, st
    return q, scales


_FP8_WS: dict = {}


def fp8_linear(x: torch.Tensor, w_q: torch.Tensor, w_scale: torch.Tensor,
               bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out = x @ dequant(w_q).T via the fp8 weight-streaming kernel
    (M <= 256): per-token-group activation quant + block-scale fp8
    MFMA. Weights stream at 1 B/elem — ~2x the bf16 decode rate."""
    M, K = x.shape
    N = w_q.shape[0]
    aq, _, ast = per_token_group_quant_fp8(x.contiguous(),
                                           transposed=True)
    splitk = _quant_splitk(N, K, 128)
    need = splitk * M * N
    key = x.device.index or 0
    ws = _FP8_WS.get(key)
    if ws is None or ws.numel() < need:
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError("fp8 workspace grown during graph capture")
        ws = torch.empty(need, dtype=torch.float32, device=x.device)
        _FP8_WS[key] = ws
    out = torch.empty(M, N, dtype=x.dtype, device=x.device)
    _gpu_kernels().fp8_skinny_gemm(
        out, aq.view(torch.uint8), ast, w_q.view(torch.uint8),
        w_scale.contiguous(),
        bias.float() if bias is not None else None, ws, splitk)
    return out


_IDENT: dict = {}


def _identity_tables(device, m_pad: int, block: int):
    """Routing tables that make the grouped MoE GEMM a plain dense
    GEMM: sorted_ids = arange (row i of the batch is 'pair' i, topk=1),
    every block belongs to expert 0. Cached per (device, m_pad) — the
    graph warmup pass populates the cache so capture never allocates."""
    key = (device.index or 0, m_pad, block)
    ent = _IDENT.get(key)
    if ent is None:
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError("identity tables built during graph capture")
        ids = torch.arange(m_pad, dtype=torch.int32, device=device)
        blocks = torch.zeros(m_pad // block, dtype=torch.int32,
                             device=device)
        n_post = torch.full((1,), m_pad, dtype=torch.int32, device=device)
        ent = (ids, blocks, n_post)
        _IDENT[key] = ent
    return ent


def fp8_prefill_linear(x: torch.Tensor, w_q: torch.Tensor,
                       w_scale: torch.Tensor,
                       bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Dense fp8 GEMM for M > 256: the grouped MoE fp8 kernel (wide
    BM64xBN256 prefill tile) with identity routing — weights stay e4m3,
    no per-call dequant materialization."""
    M, K = x.shape
    N = w_q.shape[0]
    aq, as_ = per_token_group_quant_fp8(x.contiguous())
    m_pad = (M + 63) // 64 * 64
    ids, blocks, n_post = _identity_tables(x.device, m_pad, 64)
    out_pad = torch.empty(m_pad, N, dtype=x.dtype, device=x.device)
    _gpu_kernels().moe_gemm_fp8(
        out_pad, aq.view(torch.uint8), as_,
        w_q.view(torch.uint8).view(1, N, K),
        w_scale.contiguous().view(1, w_scale.shape[0], w_scale.shape[1]),
        ids, blocks, n_post, None, M, 1, 164, False)
    out = out_pad.narrow(0, 0, M)
    if bias is not None:
        out = out.add_(bias)
    return out


def int4_prefill_linear(x: torch.Tensor, wq4: torch.Tensor,
                        sb: torch.Tensor,
                        bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Dense int4 (w4a16) GEMM for M > 256 via the grouped MoE int4
    kernel with identity routing — packed nibbles stream directly."""
    M, K2 = x.shape[0], wq4.shape[1]
    N = wq4.shape[0]
    m_pad = (M + 63) // 64 * 64
    ids, blocks, n_post = _identity_tables(x.device, m_pad, 64)
    out_pad = torch.empty(m_pad, N, dtype=x.dtype, device=x.device)
    _gpu_kernels().moe_gemm_int4(
        out_pad, x.contiguous(), wq4.view(1, N, K2),
        sb.view(1, N, -1, 2).contiguous() if sb.dim() == 3 else sb,
        ids, blocks, n_post, None, M, 1, 64, False)
    out = out_pad.narrow(0, 0, M)
    if bias is not None:
        out = out.add_(bias)
    return out


def fused_moe_fp8(x: torch.Tensor, w13: torch.Tensor, w13_scale,
                  w2: torch.Tensor, w2_scale,
                  topk_weights: torch.Tensor, topk_ids: torch.Tensor,
                  expert_start: int = 0) -> torch.Tensor:
    """fp8 grouped-GEMM MoE: same align/sum pipeline as fused_moe with
    block-scale fp8 GEMMs; expert weights stay e4m3-resident."""
    T, K = x.shape
    E_local, two_i, _ = w13.shape
    topk = topk_ids.shape[1]
    n_pairs = T * topk
    # same tile heuristic as the bf16 path (164 = BM64 x BN256 prefill)
    rpe = n_pairs / max(1, E_local)
    if n_pairs >= 4096:
        align_m, gemm_m = 64, 164
    elif rpe < 12:
        align_m = gemm_m = 16
    elif rpe < 40:
        align_m = gemm_m = 32
    else:
        align_m = gemm_m = 64
    cap = n_pairs + E_local * (align_m - 1) + 1
    max_blocks = (n_pairs + align_m - 1) // align_m + E_local
    dev = x.device
    k = _gpu_kernels()
    ids32 = topk_ids.int().contiguous()
    sorted_ids = torch.empty(cap, dtype=torch.int32, device=dev)
    expert_blocks = torch.empty(max_blocks, dtype=torch.int32, device=dev)
    n_post = torch.empty(1, dtype=torch.int32, device=dev)
    k.moe_align(ids32, E_local, expert_start, align_m, sorted_ids,
                expert_blocks, n_post)
    rows_pad = cap - 1 + align_m
    aq, as_ = per_token_group_quant_fp8(x.contiguous())
    inter1 = torch.empty(rows_pad, two_i, dtype=x.dtype, device=dev)
    k.moe_gemm_fp8(inter1, aq.view(torch.uint8), as_,
                   w13.view(torch.uint8), w13_scale.contiguous(),
                   sorted_ids, expert_blocks, n_post, None, n_pairs, topk,
                   gemm_m, False)
    act = silu_and_mul(inter1)
    actq, act_s = per_token_group_quant_fp8(act)
    pair_out = x.new_zeros(n_pairs, K)
    k.moe_gemm_fp8(pair_out, actq.view(torch.uint8), act_s,
                   w2.view(torch.uint8), w2_scale.contiguous(),
                   sorted_ids, expert_blocks, n_post,
                   topk_weights.float().contiguous(), n_pairs, topk,
                   gemm_m, True)
    out = torch.empty(T, K, dtype=x.dtype, device=dev)
    k.moe_sum(out, pair_out, topk)
    return out


# --------------------------------------------------------------- gdn
def gdn_conv_update(x: torch.Tensor, weight: torch.Tensor,
                    conv_state: torch.Tensor,
                    slots: torch.Tensor) -> torch.Tensor:
    """Batched causal-conv1d decode step: x [B, C] one token per seq,
    conv_state pool rows indexed by ``slots`` roll in place."""
    out = torch.empty_like(x)
    _gpu_kernels().gdn_conv_update(out, x, weight, conv_state, slots)
    return out


def gdn_decode(qn: torch.Tensor, kn: torch.Tensor, v: torch.Tensor,
               g: torch.Tensor, beta: torch.Tensor, state: torch.Tensor,
               slots: torch.Tensor) -> torch.Tensor:
    """Batched fused recurrent gated-delta-rule step (one token per
    seq). qn/kn [B, Hv, 128] fp32 (normalized, q pre-scaled), v [B, Hv,
    Dv] fp32; state pool [slots, Hv, Dv, 128] fp32 updated in place."""
    B, Hv, Dv = v.shape
    o = torch.empty(B, Hv, Dv, dtype=torch.bfloat16, device=v.device)
    _gpu_kernels().gdn_decode(o, qn.contiguous(), kn.contiguous(),
                              v.contiguous(), g.contiguous(),
                              beta.contiguous(), state, slots)
    return o


def gdn_chunk_prefill(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                      g: torch.Tensor, beta: torch.Tensor,
                      states: torch.Tensor, scale: float) -> torch.Tensor:
    """Fused WY chunk-parallel gated delta rule over a padded batch
    (one launch per layer; replaces ~25 torch launches per 256-token
    chunk). q/k [B, T, Hk, 128], v [B, T, Hv, 128], g/beta [B, T, Hv]
    fp32, states [B, Hv, 128, 128] fp32 updated IN PLACE. Falls back
    to the torch oracle off-GPU or for non-128 head dims."""
    B, T, Hk, Dk = q.shape
    Hv, Dv = v.shape[2], v.shape[3]
    if not (q.is_cuda and has_kernels() and Dk == 128 and Dv == 128
            and Hv % Hk == 0):
        from gllm_amd.ops import gdn_ref
        return gdn_ref.gated_delta_rule_chunked_batched(
            q, k, v, g, beta, scale, states)
    Tp = (T + 63) // 64 * 64
    if Tp != T:  # zero padding rows carry g = 0, beta = 0 -> inert
        pad = (0, 0, 0, 0, 0, Tp - T)
        q = torch.nn.functional.pad(q, pad)
        k = torch.nn.functional.pad(k, pad)
        v = torch.nn.functional.pad(v, pad)
        g = torch.nn.functional.pad(g, (0, 0, 0, Tp - T))
        beta = torch.nn.functional.pad(beta, (0, 0, 0, Tp - T))
    o = torch.empty(B, Tp, Hv, Dv, dtype=torch.bfloat16, device=q.device)
    _gpu_kernels().gdn_chunk_prefill(
        o, q.to(torch.bfloat16).contiguous(),
        k.to(torch.bfloat16).contiguous(),
        v.to(torch.bfloat16).contiguous(),
        g.float().contiguous(), beta.float().contiguous(),
        states, float(scale))
    return o[:, :T]


def rmsnorm_gated(x: torch.Tensor, z: torch.Tensor, weight: torch.Tensor,
                  eps: float) -> torch.Tensor:
    """out = rmsnorm(x) * w * silu(z) (fused, GPU)."""
    if not x.is_cuda:
        from gllm_amd.ops import gdn_ref
        return gdn_ref.rmsnorm_gated(x, z, weight, eps)
    out = torch.empty_like(x)
    _gpu_kernels().rmsnorm_gated(out, x.contiguous(), z.contiguous(),
                                 weight, eps)
    return out


def int4_linear(x: torch.Tensor, wq4: torch.Tensor, sbt: torch.Tensor,
                group: int,
                bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out = x @ dequant(wq4).T via the fused-dequant int4 skinny GEMM
    (M <= 256): packed nibbles stream at 0.5 B/elem. ``sbt`` is the
    TRANSPOSED (scale, bias) bank [K/group, 2, N] (lane-contiguous
    staging; repack_canonical builds it)."""
    M, K = x.shape
    N = wq4.shape[0]
    splitk = _quant_splitk(N, K, 256)
    need = splitk * M * N
    key = x.device.index or 0
    ws = _FP8_WS.get(key)  # shares the fp32 partial workspace pool
    if ws is None or ws.numel() < need:
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError("int4 workspace grown during graph capture")
        ws = torch.empty(need, dtype=torch.float32, device=x.device)
        _FP8_WS[key] = ws
    out = torch.empty(M, N, dtype=x.dtype, device=x.device)
    _gpu_kernels().int4_skinny_gemm(
        out, x.contiguous(), wq4, sbt,
        bias.float() if bias is not None else None, ws, group)
    return out


def fused_moe_int4(x: torch.Tensor, w13_c, w13_sb, w2_c, w2_sb,
                   topk_weights: torch.Tensor, topk_ids: torch.Tensor,
                   expert_start: int = 0) -> torch.Tensor:
    """int4 (w4a16) grouped-GEMM MoE: packed-nibble expert banks with
    in-fragment dequant — no bf16 materialization at all."""
    T, K = x.shape
    E_local, two_i, _ = w13_c.shape
    topk = topk_ids.shape[1]
    n_pairs = T * topk
    rpe = n_pairs / max(1, E_local)
    block_m = 16 if rpe < 12 else (32 if rpe < 40 else 64)
    cap = n_pairs + E_local * (block_m - 1) + 1
    max_blocks = (n_pairs + block_m - 1) // block_m + E_local
    dev = x.device
    k = _gpu_kernels()
    ids32 = topk_ids.int().contiguous()
    sorted_ids = torch.empty(cap, dtype=torch.int32, device=dev)
    expert_blocks = torch.empty(max_blocks, dtype=torch.int32, device=dev)
    n_post = torch.empty(1, dtype=torch.int32, device=dev)
    k.moe_align(ids32, E_local, expert_start, block_m, sorted_ids,
                expert_blocks, n_post)
    rows_pad = cap - 1 + block_m
    inter1 = torch.empty(rows_pad, two_i, dtype=x.dtype, device=dev)
    k.moe_gemm_int4(inter1, x.contiguous(), w13_c, w13_sb, sorted_ids,
                    expert_blocks, n_post, None, n_pairs, topk, block_m,
                    False)
    act = silu_and_mul(inter1)
    pair_out = x.new_zeros(n_pairs, K)
    k.moe_gemm_int4(pair_out, act, w2_c, w2_sb, sorted_ids,
                    expert_blocks, n_post,
                    topk_weights.float().contiguous(), n_pairs, topk,
                    block_m, True)
    out = torch.empty(T, K, dtype=x.dtype, device=dev)
    k.moe_sum(out, pair_out, topk)
    return out


# --------------------------------------------------------------- sampling
def topk_topp_filter(probs: torch.Tensor, top_ks: torch.Tensor,
                     top_ps: torch.Tensor,
                     min_ps: Optional[torch.Tensor] = None):
    """In-place fused top-k/top-p/min-p filter + renormalize on [B, V]
    fp32 probs (GPU kernel; sorting-free 3-level radix select). CPU
    callers use the torch sort composite in layers/sampler.py."""
    assert probs.is_cuda
    _gpu_kernels().topk_topp_filter(
        probs, top_ks.int(), top_ps.float(),
        min_ps.float() if min_ps is not None else None)
    return probs


# --------------------------------------------------------------- mla
def apply_penalty_pool(logits, mask_pool, slots, penalties):
    """In-place repetition penalty against the persistent uint8 mask
    pool (GPU kernel; CPU callers use the inline torch math in
    layers/sampler.py)."""
    assert logits.is_cuda
    _gpu_kernels().apply_repetition_penalty(logits, mask_pool, slots,
                                            penalties)
    return logits


def cache_latent(k, k_cache, slot_mapping):
    """Scatter the absorbed-MLA latent row [T, 1, lora+rope] into the
    paged latent cache (the v 'cache' is a view of its first lora dims,
    so one write covers both). Reference concat_and_cache_mla
    (cache_kernels.py:161)."""
    if k.is_cuda:
        if k_cache.shape[-1] == 576:
            _gpu_kernels().cache_latent(
                k.reshape(k.shape[0], -1), k_cache, slot_mapping)
        else:  # non-standard latent width: plain K/V scatter, twice
            _gpu_kernels().reshape_and_cache(k, k, k_cache, k_cache,
                                             slot_mapping)
        return
    page_size = k_cache.shape[1]
    pages = torch.div(slot_mapping, page_size, rounding_mode="floor")
    offs = slot_mapping % page_size
    k_cache[pages, offs] = k.to(k_cache.dtype)


_MLA_GPU_WARNED = False


def mla_paged_attention(q, k_cache, v_cache, block_table, seq_lens,
                        query_start_loc, scale, topk_positions=None,
                        seq_lens_cpu=None, query_start_loc_cpu=None):
    """Varlen causal attention with asymmetric head dims (MLA).

    GPU + absorbed layout (Hkv=1, 576-dim latent) -> the gfx950 MQA
    MFMA kernel (one kernel serves decode w/ split-KV, chunked prefill
    and mixed batches — reference attention.py:366-446,653-925 roles).
    DSA sparse selection (topk_positions) and the non-absorbed debug
    layout stay on the torch path."""
    global _MLA_GPU_WARNED
    if (q.is_cuda and topk_positions is None and k_cache.shape[2] == 1
            and q.shape[-1] == 576 and v_cache.shape[-1] == 512
            and q.dtype == torch.bfloat16):
        qsl_h = query_start_loc_cpu or query_start_loc.tolist()
        lens_h = seq_lens_cpu or seq_lens.tolist()
        max_q = max((qsl_h[i + 1] - qsl_h[i] for i in range(len(lens_h))),
                    default=1)
        max_s = max(lens_h, default=1)
        T, H = q.shape[0], q.shape[1]
        out = torch.empty(T, H, 512, dtype=q.dtype, device=q.device)
        qsl_i = query_start_loc.int() \
            if query_start_loc.dtype != torch.int32 else query_start_loc
        _gpu_kernels().mla_paged_attention(
            out, q.contiguous(), k_cache, block_table, seq_lens, qsl_i,
            max_q, scale, max_s)
        return out
    if q.is_cuda and not _MLA_GPU_WARNED:
        from gllm_amd.logger import logger
        logger.warning("MLA attention falls back to the torch path on "
                       "GPU (sparse/non-absorbed layout)")
        _MLA_GPU_WARNED = True
    return torch_ref.mla_paged_attention(
        q, k_cache, v_cache, block_table, seq_lens, query_start_loc,
        scale, topk_positions=topk_positions, seq_lens_cpu=seq_lens_cpu,
        query_start_loc_cpu=query_start_loc_cpu)


# --------------------------------------------------------------- gemm
_SKINNY_WS: dict = {}
SKINNY_MAX_M = 256


def _skinny_splitk(M: int, N: int, K: int) -> int:
    # v2 kernel grid is (N/64, splitk) — M-blocks live INSIDE one
    # workgroup, so the fill target counts only N tiles
    n_wg = -(-N // 64)
    s = 1
    while s < 16 and n_wg * s < 512 and (K // (s * 2)) >= 64:
        s *= 2
    k_slice = ((-(-K // s)) + 63) // 64 * 64
    return -(-K // k_slice)


def _quant_splitk(N: int, K: int, bk: int) -> int:
    """splitk for the quant skinny GEMMs (fp8 bk=128, int4 bk=256):
    deepest split that still leaves >= 8 ring stages per block, with
    the grid capped near chip size (measured sweep, profiles/)."""
    n_wg = -(-N // 64)
    s = 1
    while (s < 16 and n_wg * (s * 2) <= 1024
           and (K // bk) // (s * 2) >= 8):
        s *= 2
    k_slice = ((-(-K // s)) + bk - 1) // bk * bk
    return -(-K // k_slice)


def skinny_gemm(x: torch.Tensor, w: torch.Tensor,
                bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out = x @ w.T via the gfx950 weight-streaming kernel (M<=256-ish)."""
    import os
    M, K = x.shape
    N = w.shape[0]
    splitk = int(os.environ.get("SK_SPLITK", "0")) or \
        _skinny_splitk(M, N, K)
    need = splitk * M * N
    key = x.device.index or 0
    ws = _SKINNY_WS.get(key)
    if ws is None or ws.numel() < need:
        if torch.cuda.is_current_stream_capturing():
            # growing the cached workspace mid-capture would free the
            # buffer an earlier-captured graph writes (the r1 replay
            # fault class); warmup must size it first
            raise RuntimeError(
                "skinny_gemm workspace grown during graph capture — "
                "run an eager warmup at the largest bucket first")
        ws = torch.empty(need, dtype=torch.float32, device=x.device)
        _SKINNY_WS[key] = ws
    out = torch.empty(M, N, dtype=x.dtype, device=x.device)
    _gpu_kernels().skinny_gemm(out, x, w, None, ws, splitk)
    if bias is not None:
        out += bias
    return out


def _use_skinny(M: int, N: int, K: int) -> bool:
    """Measured dispatch rule (scripts/gemm_sweep.py on MI355X r01):
    the skinny kernel beats hipBLASLt on K-deep reductions at any decode
    M (down_proj: 1.9 -> 4.1 TB/s) and on every N<=8k shape once M>64
    (library tiles collapse to ~1.1-1.6 TB/s there); the library keeps
    wide-N shapes (gate_up, lm_head) and small-M small-K projections."""
    import os
    if os.environ.get("GLLM_DISABLE_SKINNY"):
        return False
    max_m = int(os.environ.get("GLLM_SKINNY_MAX_M", "0")) or SKINNY_MAX_M
    if K % 64 != 0 or N < 1024 or M > max_m:
        return False
    # MB>=2 under capture: r1 faulted with dynamic LDS; the kernel now
    # uses static LDS and captures cleanly (scripts/graph_skinny_repro)
    if K >= 2 * N:
        return True
    return M > 64 and N <= 8192


def linear(x: torch.Tensor, w: torch.Tensor,
           bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """GEMM dispatch: the skinny weight-streaming kernel where measured
    faster, hipBLASLt otherwise."""
    import torch.nn.functional as F
    if (x.is_cuda and x.dtype == torch.bfloat16 and x.dim() == 2
            and x.is_contiguous()
            and _use_skinny(x.shape[0], w.shape[0], w.shape[1])):
        return skinny_gemm(x, w, bias)
    return F.linear(x, w, bias)


# --------------------------------------------------------------- layer norm
def layernorm_f32(x: torch.Tensor, w: torch.Tensor, b, eps: float,
                  dtype) -> torch.Tensor:
    """h = LayerNorm(x) with weight and optional bias (``b`` None =
    weight only); x is the fp32 residual stream, h comes out in
    ``dtype`` (the dtype of w and b)."""
    if x.is_cuda:
        out = torch.empty(x.shape, dtype=dtype, device=x.device)
        _seq_kernels().layernorm_f32(out, x, w, b, eps)
        return out
    return torch_ref.layernorm_f32(x, w, b, eps, dtype)


def residual_layernorm(x: torch.Tensor, y: torch.Tensor, w_post, b_post,
                       eps: float, pre=None, gate=None):
    """x (fp32, in place) += LN_post(y); with ``pre`` = (weight, bias)
    also returns LN_pre(x) in y's dtype — one launch per layer boundary
    of a sandwich-norm decoder. Biases may be None. ``gate`` ([rows,
    width] logits, row views allowed): LN_post sees y * sigmoid(gate),
    the product formed in fp32 inside the same launch."""
    if x.is_cuda:
        h = None
        if pre is not None:
            h = torch.empty(x.shape, dtype=y.dtype, device=x.device)
            _seq_kernels().residual_layernorm(x, y, w_post, b_post, h,
                                              pre[0], pre[1], eps, gate)
        else:
            _seq_kernels().residual_layernorm(x, y, w_post, b_post, None,
                                              None, None, eps, gate)
        return h
    return torch_ref.residual_layernorm(x, y, w_post, b_post, eps, pre,
                                        gate)


def stream_rmsnorm(x: torch.Tensor, y, w_post, eps: float,
                   mult: float = 1.0, y_scale: float = 1.0, y2=None,
                   add=None, pre_w=None):
    """One launch per sublayer boundary of an RMS sandwich-norm decoder
    over an fp32 stream x (in place):
        x += mult * RMSnorm(y_scale * (y + y2)) * w_post   (y given)
        x += add                                           (add: fp32 [width])
        returns RMSnorm(x) * pre_w in pre_w's dtype        (pre_w given)
    y / y2 may be row views; statistics and sums are fp32."""
    if x.is_cuda:
        h = None
        if pre_w is not None:
            h = torch.empty(x.shape, dtype=pre_w.dtype, device=x.device)
        _seq_kernels().stream_rmsnorm(x, y, y2, w_post, add, h, pre_w,
                                      float(eps), float(mult),
                                      float(y_scale))
        return h
    return torch_ref.stream_rmsnorm(x, y, w_post, eps, mult, y_scale, y2,
                                    add, pre_w)


def gated_act_mul(x: torch.Tensor, act: str = "silu") -> torch.Tensor:
    """x [rows, 2d] = gate | up -> act(gate) * up with act "silu" or
    "gelu_tanh"; any d, rows may be strided (bf16 or fp32)."""
    assert act in ("silu", "gelu_tanh")
    if x.is_cuda:
        out = torch.empty(x.shape[0], x.shape[1] // 2, dtype=x.dtype,
                          device=x.device)
        _seq_kernels().gated_act_mul(out, x, 0 if act == "silu" else 1)
        return out
    if act == "silu":
        return torch_ref.silu_and_mul(x)
    return torch_ref.gelu_tanh_and_mul(x)


def tanh_rows(x: torch.Tensor) -> torch.Tensor:
    """tanh of x [rows, n] (a column block of a wider buffer is fine),
    contiguous result in x's dtype."""
    if x.is_cuda:
        out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
        _seq_kernels().tanh_rows(out, x)
        return out
    return torch.tanh(x.float()).to(x.dtype)


def sigmoid_group_topk(logits: torch.Tensor, correction, topk: int,
                       n_group: int = 1, keep: int = 1,
                       scale: float = 1.0):
    """Sigmoid router with a selection-only correction and group
    limits, one kernel on the GPU. logits fp32 [T, E]; returns (weights
    fp32 [T, topk], ids int32 [T, topk]). See torch_ref for the rule."""
    if logits.is_cuda:
        T = logits.shape[0]
        weights = torch.empty(T, topk, dtype=torch.float32,
                              device=logits.device)
        ids = torch.empty(T, topk, dtype=torch.int32, device=logits.device)
        _seq_kernels().sigmoid_group_topk(weights, ids, logits, correction,
                                          int(n_group), int(keep),
                                          float(scale))
        return weights, ids
    return torch_ref.sigmoid_group_topk(logits, correction, topk, n_group,
                                        keep, scale)


# --------------------------------------------------------------- windowed attn
def qk_norm_rope_store(q, k, v, q_w, k_w, positions, slot_mapping, freqs,
                       mag, rot_dims, k_cache, v_cache, H, G, D, Dv, eps,
                       half_layout=False, norm_last=False, do_norm=True,
                       v_freqs=None, norm_span=False, v_unit=False,
                       q_out=None):
    """Fused per-head q/k RMS norm, rotary (per-pair frequency table
    ``freqs`` fp64, cos/sin scaled by ``mag``) and paged K/V store.
    q [T, H*D] is updated in place (may be a column slice of a merged
    projection); k/v None = the layer reads another's cache.

    ``q_w``/``k_w`` None: unit-RMS heads without a weight.
    ``half_layout``: dimension i rotates with i + rot_dims/2 (the
    default pairs 2i with 2i+1). ``norm_last``: rotate, then norm.
    ``v`` may be ``k`` itself (values = keys as projected).
    ``do_norm`` False: rotary and store only. ``v_freqs`` (fp64
    [Dv/2]): each value row is turned by its own position over all of
    Dv (same pair layout) on its way into the cache.
    ``norm_span``: one RMS over all heads of a token's q (and of its k)
    with weights that cover the row ([H*D], [G*D]). ``v_unit``: each
    value head is divided by its RMS (eps inside the root, no weight)
    before it is stored. ``q_out`` ([T, H*D]): the prepared queries go
    there and q stays as it came (required with ``norm_span``)."""
    if q.is_cuda:
        _seq_kernels().qk_norm_rope_store(
            q, k, v, q_w, k_w, positions, slot_mapping, freqs, mag,
            rot_dims, k_cache, v_cache, H, G, D, Dv, eps,
            bool(half_layout), bool(norm_last), bool(do_norm), v_freqs,
            bool(norm_span), bool(v_unit), q_out)
        return
    torch_ref.qk_norm_rope_store(q, k, v, q_w, k_w, positions,
                                 slot_mapping, freqs, mag, rot_dims,
                                 k_cache, v_cache, H, G, D, Dv, eps,
                                 half_layout, norm_last, do_norm, v_freqs,
                                 norm_span, v_unit, q_out)


def rotate_scale_rows(x, positions, freqs, heads, D, sign=1.0, scale=1.0,
                      half_layout=False, out=None) -> torch.Tensor:
    """Turn the pairs of every head row of x [T, heads*D] by
    sign * position * freqs[m] and scale the result (sign -1 undoes the
    turn that rotated values carry). ``out`` may be a column block of a
    wider buffer."""
    if x.is_cuda:
        if out is None:
            out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
        _seq_kernels().rotate_scale_rows(out, x, positions, freqs, heads, D,
                                         float(sign), float(scale),
                                         bool(half_layout))
        return out
    return torch_ref.rotate_scale_rows(x, positions, freqs, heads, D, sign,
                                       scale, half_layout, out)


def rms_weight_store(x, w, eps, cache=None, slot_mapping=None):
    """x / rms(x) * w per row (fp32 inside, x's dtype out); with
    ``cache`` [pages, page, 1, n] the normed rows are also scattered
    into their paged slots (a cached low-rank latent)."""
    if x.is_cuda:
        out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
        _seq_kernels().rms_weight_store(out, x, w, eps, cache, slot_mapping)
        return out
    return torch_ref.rms_weight_store(x, w, eps, cache, slot_mapping)


# --------------------------------------------------------------- streams
def hyper_streams(xs, y=None, y2=None, gate=None, mix=None, out_w=None,
                  read=None, dtype=None):
    """Hyper-connection residual xs [S, T, W] fp32.

    Write (``y`` given, in place): x_t <- sum_s mix[s, t] x_s +
    out_w[t] * (y + sigmoid(gate) * y2), all streams from the old ones;
    y2 / gate ([T, 1] logits) optional. Read (``read`` = (in_w [S],
    gain [1], eps)): returns gain * u / rms(u) in ``dtype`` with
    u = sum_s in_w[s] x_s — of the updated streams when both are asked
    for (one launch per sublayer boundary)."""
    if xs.is_cuda:
        h = None
        in_w = gain = None
        eps = 0.0
        if read is not None:
            in_w, gain, eps = read
            h = torch.empty(xs.shape[1:], dtype=dtype, device=xs.device)
        _seq_kernels().hyper_streams(xs, y, y2, gate, mix, out_w, h, in_w,
                                     gain, eps)
        return h
    return torch_ref.hyper_streams(xs, y, y2, gate, mix, out_w, read, dtype)


# --------------------------------------------------------------- minGRU
def mingru_varlen(zx, gp, state, slots, has_init, query_start_loc,
                  scale=1.0, max_query_len=0, out=None) -> torch.Tensor:
    """Ragged minGRU (prompt portions and decode tokens in one
    launch): zx [T, 2C] update-gate | candidate pre-activations, gp
    [T, C] read-out gate logits, fp32 state [slots, C] in place.
    Returns scale * S_t * silu(gp_t) in zx's dtype ([T, C]; ``out`` may
    be a column block of a wider buffer)."""
    if zx.is_cuda:
        if out is None:
            out = torch.empty(gp.shape, dtype=zx.dtype, device=zx.device)
        _seq_kernels().mingru_varlen(out, zx, gp, state, slots, has_init,
                                     query_start_loc, float(scale),
                                     int(max_query_len))
        return out
    return torch_ref.mingru_varlen(zx, gp, state, slots, has_init,
                                   query_start_loc, scale, out)


def clamp_swiglu(x: torch.Tensor, limit: float,
                 alpha: float = 1.702) -> torch.Tensor:
    """x [rows, 2d] = gate | up -> min(g, limit) * sigmoid(alpha g) *
    (clamp(u, -limit, limit) + 1)."""
    if x.is_cuda:
        out = torch.empty(x.shape[0], x.shape[1] // 2, dtype=x.dtype,
                          device=x.device)
        _seq_kernels().clamp_swiglu(out, x, float(limit), float(alpha))
        return out
    return torch_ref.clamp_swiglu(x, limit, alpha)


def window_attention(q, gate, k_cache, v_cache, block_table, seq_lens,
                     query_start_loc, scale, window=0, keep_first=0,
                     sink=False, max_query_len=0, sinks=None,
                     softcap=0.0, out=None) -> torch.Tensor:
    """Ragged paged attention over K [pages, page, G, D] / V [.., Dv]:
    sliding window with kept first tokens, optional softmax sink (+1 in
    the denominator; ``sinks`` fp32 [H]: exp(sinks[h]) instead), tanh
    score cap (``softcap`` > 0: cap * tanh(s / cap)) and fused sigmoid
    output gate. K and V may be the same tensor (attention over a
    cached latent). Returns [T, H*Dv]; ``out`` may be a column block
    of a wider buffer.

    Batches that hold prompt portions (``max_query_len`` > 1) in bf16
    with D == Dv in {64, 128} run the MFMA tile kernel shared with
    paged_attention (128 query rows per workgroup, K/V streamed through
    LDS); decode-only bf16 batches with an instantiated (D, GQA ratio)
    run the split-KV decode kernels; fp32 and every other head geometry
    run the generic one-workgroup-per-(token, head) kernel."""
    if q.is_cuda:
        T = q.shape[0]
        D, Dv = k_cache.shape[3], v_cache.shape[3]
        H = q.shape[1] // D
        if out is None:
            out = torch.empty(T, H * Dv, dtype=q.dtype, device=q.device)
        if (max_query_len > 1 and q.dtype == torch.bfloat16 and D == Dv
                and D in (64, 128)):
            _seq_kernels().window_attention_mfma(
                out, q, gate, k_cache, v_cache, block_table, seq_lens,
                query_start_loc, max_query_len, scale, window, keep_first,
                sink, sinks, softcap)
            return out
        if (max_query_len == 1 and q.dtype == torch.bfloat16 and D == Dv
                and _seq_kernels().window_attention_decode(
                    out, q, gate, k_cache, v_cache, block_table, seq_lens,
                    scale, window, keep_first, sink, sinks, softcap)):
            # decode-only batch on the split-KV kernels shared with
            # paged_attention (one workgroup per GQA group and KV split)
            return out
        _seq_kernels().window_attention(
            out, q, gate, k_cache, v_cache, block_table, seq_lens,
            query_start_loc, scale, window, keep_first, sink, sinks,
            softcap)
        return out
    res = torch_ref.window_attention(q, gate, k_cache, v_cache,
                                     block_table, seq_lens,
                                     query_start_loc, scale, window,
                                     keep_first, sink, sinks, softcap)
    if out is not None:
        out.copy_(res)
        return out
    return res


# --------------------------------------------------------------- talking heads
def talking_attention(q, k_cache, v_cache, block_table, seq_lens,
                      query_start_loc, scale, talk, sink=None,
                      max_query_len=0) -> torch.Tensor:
    """Ragged paged causal attention with cross-head score mixing:
    s_g = scale * q_g . k_kv(g) for all H heads, s'_h = sum_g
    talk[h, g] s_g, softmax over the keys per head with exp(sink[h])
    added to the denominator (``sink`` None: plain softmax), output
    head h = weights . v_kv(h). K [pages, page, G, D], V [.., Dv];
    talk [H, H] and sink [H] fp32. Returns [T, H*Dv].

    All heads of a query are handled together (the mix couples them).
    bf16 batches with prompt portions and D == Dv a multiple of 32
    run the MFMA tile kernel; bf16 decode-only batches the split-KV
    kernel; fp32 and other shapes the generic kernel."""
    if q.is_cuda:
        T = q.shape[0]
        D, Dv = k_cache.shape[3], v_cache.shape[3]
        H = q.shape[1] // D
        out = torch.empty(T, H * Dv, dtype=q.dtype, device=q.device)
        _seq_kernels().talking_attention(
            out, q, k_cache, v_cache, block_table, seq_lens,
            query_start_loc, scale, talk, sink, max_query_len)
        return out
    return torch_ref.talking_attention(q, k_cache, v_cache, block_table,
                                       seq_lens, query_start_loc, scale,
                                       talk, sink)


# --------------------------------------------------------------- activations
def xielu(x: torch.Tensor, a_pos: float, a_neg: float) -> torch.Tensor:
    """xIELU: z > 0 -> a_pos z^2 + z/2, else a_neg (e^z - 1 - z) + z/2."""
    if x.is_cuda:
        out = torch.empty_like(x)
        _seq_kernels().xielu(out, x, a_pos, a_neg)
        return out
    return torch_ref.xielu(x, a_pos, a_neg)


def relu2(x: torch.Tensor) -> torch.Tensor:
    """max(x, 0)^2."""
    if x.is_cuda:
        out = torch.empty_like(x)
        _seq_kernels().relu2(out, x)
        return out
    return torch_ref.relu2(x)


# --------------------------------------------------------------- delta rule
def causal_conv_silu(x, w, conv_state, slots, has_init, query_start_loc,
                     activation=True, max_query_len=0):
    """Ragged short causal conv + silu (``activation`` False: the plain
    convolution); rolls ``conv_state`` rows ``slots`` in place. x may be
    a column slice of a merged projection. ``max_query_len`` == 1
    (decode-only batch): the state is rolled by the same launch."""
    if x.is_cuda:
        out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
        _seq_kernels().causal_conv_silu(out, x, w, conv_state, slots,
                                        has_init, query_start_loc,
                                        bool(activation),
                                        int(max_query_len))
        return out
    from gllm_amd.ops import gdn_ref
    return gdn_ref.causal_conv_silu(x, w, conv_state, slots, has_init,
                                    query_start_loc, activation)


def delta_rule_varlen(q, k, v, a, b, A_log, dt_bias, state, slots,
                      has_init, query_start_loc, q_scale,
                      max_query_len=0) -> torch.Tensor:
    """Ragged gated delta rule (prompt portions and decode tokens in one
    launch); fp32 state [slots, H, Dk, Dv] in place; returns fp32
    [T, H, Dv]. ``max_query_len`` == 1 (decode-only batch) keeps the
    operands in registers; anything else stages token tiles through
    LDS — same arithmetic per token either way."""
    if q.is_cuda:
        H, _, Dv = state.shape[1:]
        o = torch.empty(q.shape[0], H, Dv, dtype=torch.float32,
                        device=q.device)
        _seq_kernels().delta_rule_varlen(o, q, k, v, a, b, A_log, dt_bias,
                                         state, slots, has_init,
                                         query_start_loc, q_scale,
                                         max_query_len)
        return o
    from gllm_amd.ops import gdn_ref
    return gdn_ref.delta_rule_varlen(q, k, v, a, b, A_log, dt_bias, state,
                                     slots, has_init, query_start_loc,
                                     q_scale)


def rms_gate(o, z, w, H, eps, dtype, gate="silu", scale=1.0,
             out=None) -> torch.Tensor:
    """Per head scale * o / rms(o) * w * act(z): fp32 [T, H, Dv] ->
    [T, H*Dv]. ``w`` [Dv] serves every head, [H*Dv] gives each head its
    own; ``gate`` "silu" or "sigmoid"; ``out`` may be a column block of
    a wider buffer."""
    assert gate in ("silu", "sigmoid")
    if o.is_cuda:
        if out is None:
            out = torch.empty(o.shape[0], o.shape[1] * o.shape[2],
                              dtype=dtype, device=o.device)
        _seq_kernels().rms_gate(out, o, z, w, H, eps, gate == "sigmoid",
                                float(scale))
        return out
    from gllm_amd.ops import gdn_ref
    return gdn_ref.rms_gate(o, z, w, H, eps, dtype, gate, scale, out)


def general_delta_rule(r, k, v, w_logit, a_logit, w0, decay_scale, state,
                       slots, has_init, query_start_loc,
                       max_query_len=0) -> torch.Tensor:
    """Ragged generalized delta rule with per-channel decay and removal
    (prompt portions and decode tokens in one launch). Per head, with
    w = exp(-decay_scale * sigmoid(w_logit + w0)), a = sigmoid(a_logit),
    u = k / sqrt(|k|^2 + 1e-6):
        S <- diag(w) S - (a u)(u^T S) + k v^T,   o = S^T r
    fp32 state [slots, H, D, Dv] in place; decay, removal rate and the
    unit key are formed in fp32 from the projections. Returns fp32
    [T, H, Dv]."""
    if r.is_cuda:
        H, _, Dv = state.shape[1:]
        o = torch.empty(r.shape[0], H, Dv, dtype=torch.float32,
                        device=r.device)
        _seq_kernels().general_delta_rule(
            o, r, k, v, w_logit, a_logit, w0, float(decay_scale), state,
            slots, has_init, query_start_loc, int(max_query_len))
        return o
    from gllm_amd.ops import gdn_ref
    return gdn_ref.general_delta_rule(r, k, v, w_logit, a_logit, w0,
                                      decay_scale, state, slots, has_init,
                                      query_start_loc)


def token_shift(h, mu, state, slots, has_init, query_start_loc,
                max_query_len=0):
    """Ragged token shift h_t + (h_(t-1) - h_t) * mu: the row before a
    portion's first comes from ``state`` [slots, width] (zeros when the
    sequence starts here), which is left at the portion's last incoming
    row."""
    if h.is_cuda:
        out = torch.empty_like(h)
        _seq_kernels().token_shift(out, h, mu, state, slots, has_init,
                                   query_start_loc, int(max_query_len))
        return out
    return torch_ref.token_shift(h, mu, state, slots, has_init,
                                 query_start_loc)
