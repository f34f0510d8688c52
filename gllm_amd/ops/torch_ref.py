"""Pure-PyTorch reference implementations of every custom op.

These are (a) the CPU execution path (config 1: plumbing without a GPU)
and (b) the numerics oracle the HIP kernels are unit-tested against
(reference keeps `forward_native` impls for this purpose,
layers/layernorm.py:88-127). All math in fp32 for a stable oracle.
"""

import math
from typing import Optional

import torch


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    dtype = x.dtype
    xf = x.float()
    var = xf.pow(2).mean(-1, keepdim=True)
    out = xf * torch.rsqrt(var + eps)
    return (out * weight.float()).to(dtype)


def fused_add_rmsnorm(x: torch.Tensor, residual: torch.Tensor,
                      weight: torch.Tensor, eps: float):
    """residual += x; x = rmsnorm(residual). In-place on both args."""
    residual.add_(x)
    x.copy_(rmsnorm(residual, weight, eps))
    return x, residual


def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    d = x.shape[-1] // 2
    return (torch.nn.functional.silu(x[..., :d].float())
            * x[..., d:].float()).to(x.dtype)



def gelu_and_mul(x: torch.Tensor) -> torch.Tensor:
    """gelu(x[:, :d]) * x[:, d:] (erf-based, reference gelu_and_mul)."""
    d = x.shape[-1] // 2
    a = x[..., :d].float()
    return (torch.nn.functional.gelu(a) *
            x[..., d:].float()).to(x.dtype)

def rotary_embedding(positions: torch.Tensor, q: torch.Tensor,
                     k: torch.Tensor, head_dim: int,
                     cos_sin_cache: torch.Tensor, is_neox: bool = True):
    """In-place RoPE on q [T, Hq*D] and k [T, Hk*D].

    cos_sin_cache: [max_pos, rot_dim] laid out [cos(rot/2) | sin(rot/2)].
    """
    rot_dim = cos_sin_cache.shape[-1]
    half = rot_dim // 2
    cs = cos_sin_cache[positions].float()       # [T, rot_dim]
    cos = cs[:, :half]                          # [T, half]
    sin = cs[:, half:]
    for t in (q, k):
        T = t.shape[0]
        x = t.unflatten(-1, (-1, head_dim))
        rot = x[..., :rot_dim].float()
        if is_neox:
            x1, x2 = rot[..., :half], rot[..., half:]
            c = cos.unsqueeze(1)
            s = sin.unsqueeze(1)
            o1 = x1 * c - x2 * s
            o2 = x2 * c + x1 * s
            out = torch.cat([o1, o2], dim=-1)
        else:
            x1, x2 = rot[..., 0::2], rot[..., 1::2]
            c = cos.unsqueeze(1)
            s = sin.unsqueeze(1)
            o1 = x1 * c - x2 * s
            o2 = x2 * c + x1 * s
            out = torch.stack([o1, o2], dim=-1).flatten(-2)
        x[..., :rot_dim].copy_(out.to(t.dtype))
    return q, k


def reshape_and_cache(k: torch.Tensor, v: torch.Tensor,
                      k_cache: torch.Tensor, v_cache: torch.Tensor,
                      slot_mapping: torch.Tensor):
    """Scatter per-token K/V [T, Hkv, D] into paged caches
    [num_pages, page_size, Hkv, D] at flat slot indices."""
    page_size = k_cache.shape[1]
    pages = torch.div(slot_mapping, page_size, rounding_mode="floor")
    offs = slot_mapping % page_size
    k_cache[pages, offs] = k.to(k_cache.dtype)
    v_cache[pages, offs] = v.to(v_cache.dtype)


def paged_attention(q: torch.Tensor, k_cache: torch.Tensor,
                    v_cache: torch.Tensor, block_table: torch.Tensor,
                    seq_lens: torch.Tensor, query_start_loc: torch.Tensor,
                    scale: float, out: Optional[torch.Tensor] = None,
                    sliding_window: int = 0) -> torch.Tensor:
    """Varlen causal attention over the paged KV cache.

    q:            [T, Hq, D] — all new tokens of the batch, ragged by seq
    k/v_cache:    [num_pages, page_size, Hkv, D]
    block_table:  [B, max_pages] int — page ids per seq
    seq_lens:     [B] — TOTAL context length per seq (past + new)
    query_start_loc: [B+1] — ragged boundaries into q
    Causal offset: query token i of seq b attends to cache positions
    [0, seq_len - q_len + i].
    """
    T, Hq, D = q.shape
    Hkv = k_cache.shape[2]
    page_size = k_cache.shape[1]
    group = Hq // Hkv
    if out is None:
        out = torch.empty_like(q)
    B = seq_lens.shape[0]
    for b in range(B):
        qs, qe = int(query_start_loc[b]), int(query_start_loc[b + 1])
        q_len = qe - qs
        if q_len == 0:
            continue
        s_len = int(seq_lens[b])
        n_pages = -(-s_len // page_size)
        pages = block_table[b, :n_pages].long()
        k = k_cache[pages].reshape(-1, Hkv, D)[:s_len].float()  # [S, Hkv, D]
        v = v_cache[pages].reshape(-1, Hkv, D)[:s_len].float()
        qq = q[qs:qe].float()                                   # [L, Hq, D]
        # [Hq, L, S]
        scores = torch.einsum("lhd,shd->hls", qq,
                              k.repeat_interleave(group, dim=1)) * scale
        # causal mask with past offset
        past = s_len - q_len
        pos_q = torch.arange(q_len, device=q.device).unsqueeze(1) + past
        pos_k = torch.arange(s_len, device=q.device).unsqueeze(0)
        mask = pos_k <= pos_q                                   # [L, S]
        if sliding_window > 0:
            mask &= pos_k > (pos_q - sliding_window)
        scores.masked_fill_(~mask.unsqueeze(0), float("-inf"))
        p = torch.softmax(scores, dim=-1)
        o = torch.einsum("hls,shd->lhd", p,
                         v.repeat_interleave(group, dim=1))
        out[qs:qe] = o.to(out.dtype)
    return out


def mla_paged_attention(q: torch.Tensor, k_cache: torch.Tensor,
                        v_cache: torch.Tensor, block_table: torch.Tensor,
                        seq_lens: torch.Tensor,
                        query_start_loc: torch.Tensor,
                        scale: float,
                        topk_positions: Optional[torch.Tensor] = None,
                        seq_lens_cpu: Optional[list] = None,
                        query_start_loc_cpu: Optional[list] = None
                        ) -> torch.Tensor:
    """Varlen causal attention with asymmetric head dims (MLA):
    q/k have Dk (nope+rope), v has Dv. Same paged layout as
    paged_attention; returns [T, H, Dv].

    ``topk_positions`` (DeepSeek Sparse Attention, reference
    deepseek_v32.py:235-792): [T, topk] int per-QUERY token POSITIONS
    within the query's own sequence (-1 padded). When given, each query
    row attends ONLY to its selected positions (intersected with the
    causal mask). For topk >= seq_len the selection covers every key,
    making sparse == dense — the DSA correctness oracle."""
    T, H, Dk = q.shape
    Dv = v_cache.shape[3]
    page_size = k_cache.shape[1]
    out = torch.empty(T, H, Dv, dtype=q.dtype, device=q.device)
    B = seq_lens.shape[0]
    # host geometry (when the caller has it) avoids 2B+1 device syncs
    qsl_h = query_start_loc_cpu or query_start_loc.tolist()
    lens_h = seq_lens_cpu or seq_lens.tolist()
    for b in range(B):
        qs, qe = qsl_h[b], qsl_h[b + 1]
        q_len = qe - qs
        if q_len == 0:
            continue
        s_len = lens_h[b]
        n_pages = -(-s_len // page_size)
        pages = block_table[b, :n_pages].long()
        Hkv = k_cache.shape[2]
        k = k_cache[pages].reshape(-1, Hkv, Dk)[:s_len].float()
        v = v_cache[pages].reshape(-1, Hkv, Dv)[:s_len].float()
        if Hkv == 1 and H > 1:
            # absorbed MLA: MQA over the shared latent row
            k = k.expand(s_len, H, Dk)
            v = v.expand(s_len, H, Dv)
        qq = q[qs:qe].float()
        dev = q.device
        scores = torch.einsum("lhd,shd->hls", qq, k) * scale
        past = s_len - q_len
        pos_q = torch.arange(q_len, device=dev).unsqueeze(1) + past
        pos_k = torch.arange(s_len, device=dev).unsqueeze(0)
        mask = pos_k <= pos_q                          # [q_len, s_len]
        if topk_positions is not None:
            sel = topk_positions[qs:qe].long().to(dev)  # [q_len, topk]
            allowed = torch.zeros(q_len, s_len, dtype=torch.bool,
                                  device=dev)
            valid = (sel >= 0) & (sel < s_len)
            rows = torch.arange(q_len,
                                device=dev).unsqueeze(1).expand_as(sel)
            allowed[rows[valid], sel[valid]] = True
            mask = mask & allowed
        scores.masked_fill_(~mask.unsqueeze(0), float("-inf"))
        p = torch.softmax(scores, dim=-1)
        o = torch.einsum("hls,shd->lhd", p, v)
        out[qs:qe] = o.to(out.dtype)
    return out


def grouped_topk(scores: torch.Tensor, topk: int, n_group: int,
                 topk_group: int, renormalize: bool = True,
                 scoring: str = "softmax",
                 e_bias: Optional[torch.Tensor] = None):
    """DeepSeek grouped routing (reference: layers/moe/topk.py
    group_limited_greedy / noaux_tc). ``e_bias`` set => noaux_tc: sigmoid
    scores + bias for SELECTION, original sigmoid scores as weights."""
    T, E = scores.shape
    if scoring == "sigmoid":
        probs = scores.float().sigmoid()
    else:
        probs = torch.softmax(scores.float(), dim=-1)
    sel = probs + e_bias.float() if e_bias is not None else probs
    g = sel.view(T, n_group, E // n_group)
    if e_bias is not None:
        group_scores = g.topk(2, dim=-1)[0].sum(-1)     # noaux_tc
    else:
        group_scores = g.max(dim=-1).values
    grp_idx = group_scores.topk(topk_group, dim=-1)[1]  # [T, topk_group]
    mask = torch.zeros(T, n_group, dtype=torch.bool, device=scores.device)
    mask.scatter_(1, grp_idx, True)
    mask = mask.unsqueeze(-1).expand(T, n_group, E // n_group)
    sel = sel.masked_fill(~mask.reshape(T, E), float("-inf"))
    ids = sel.topk(topk, dim=-1)[1]
    weights = probs.gather(1, ids)
    if renormalize:
        weights = weights / weights.sum(-1, keepdim=True).clamp_min(1e-20)
    return weights, ids.to(torch.int32)


def topk_softmax(gating: torch.Tensor, topk: int, renormalize: bool = True):
    """MoE routing: softmax then top-k. Returns (weights [T,K], ids [T,K])."""
    probs = torch.softmax(gating.float(), dim=-1)
    weights, ids = torch.topk(probs, topk, dim=-1)
    if renormalize:
        weights = weights / weights.sum(-1, keepdim=True)
    return weights, ids.to(torch.int32)


def apply_repetition_penalty(logits: torch.Tensor, token_ids_per_row,
                             penalties: torch.Tensor) -> torch.Tensor:
    """logits [B, V]; token_ids_per_row: list of LongTensors; penalties [B]."""
    for i, toks in enumerate(token_ids_per_row):
        p = float(penalties[i])
        if p == 1.0 or toks.numel() == 0:
            continue
        row = logits[i]
        vals = row[toks]
        row[toks] = torch.where(vals > 0, vals / p, vals * p)
    return logits


# ------------------------------------------------------------------
# fp32-residual layer norm / windowed sink attention (CPU path + kernel
# oracle for ops.layernorm_f32, residual_layernorm, qk_norm_rope_store,
# window_attention)
def layernorm_f32(x: torch.Tensor, w: torch.Tensor, b, eps: float,
                  dtype) -> torch.Tensor:
    """LayerNorm of an fp32 row with weight and optional bias (``b``
    None: weight only), output in ``dtype``."""
    xf = x.float()
    mu = xf.mean(-1, keepdim=True)
    d = xf - mu
    var = (d * d).mean(-1, keepdim=True)
    out = d * torch.rsqrt(var + eps) * w.float()
    if b is not None:
        out = out + b.float()
    return out.to(dtype)


def residual_layernorm(x: torch.Tensor, y: torch.Tensor, w_post, b_post,
                       eps: float, pre=None, gate=None):
    """x (fp32, in place) += LN(y); returns LN_pre(x) when ``pre`` is a
    (weight, bias) pair. ``gate`` (logits, same shape as y): the norm
    sees y * sigmoid(gate)."""
    yf = y.float()
    if gate is not None:
        yf = yf * torch.sigmoid(gate.float())
    x.add_(layernorm_f32(yf, w_post, b_post, eps, torch.float32))
    if pre is None:
        return None
    return layernorm_f32(x, pre[0], pre[1], eps, y.dtype)


def stream_rmsnorm(x, y, w_post, eps, mult=1.0, y_scale=1.0, y2=None,
                   add=None, pre_w=None):
    """fp32 stream x (in place): x += mult * RMSnorm(y_scale * (y + y2))
    * w_post (skipped when ``y`` is None), then x += add (one fp32 row
    for every token); returns RMSnorm(x) * pre_w in pre_w's dtype when
    ``pre_w`` is given."""
    if y is not None:
        z = y.float()
        if y2 is not None:
            z = z + y2.float()
        z = z * y_scale
        z = z * torch.rsqrt((z * z).mean(-1, keepdim=True) + eps)
        x.add_(z * w_post.float() * mult)
    if add is not None:
        x.add_(add.float())
    if pre_w is None:
        return None
    h = x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps)
    return (h * pre_w.float()).to(pre_w.dtype)


def token_shift(h, mu, state, slots, has_init, query_start_loc):
    """Ragged token shift: row t becomes h_t + (h_(t-1) - h_t) * mu with
    h_(t-1) the row before it as it came in; a portion's first row
    looks at ``state[slot]`` (zeros for a sequence's first token), and
    the state is left at the portion's last incoming row."""
    out = torch.empty_like(h)
    qsl = query_start_loc.tolist()
    muf = mu.float()
    for b, slot in enumerate(slots.tolist()):
        s, e = qsl[b], qsl[b + 1]
        if e <= s:
            continue
        first = state[slot].to(h.dtype) if bool(has_init[b]) \
            else h.new_zeros(h.shape[1])
        prev = torch.cat([first[None], h[s:e - 1]]).float()
        cur = h[s:e].float()
        out[s:e] = (cur + (prev - cur) * muf).to(h.dtype)
        state[slot] = h[e - 1].to(state.dtype)
    return out


def gelu_tanh_and_mul(x: torch.Tensor) -> torch.Tensor:
    """gelu_tanh(x[:, :d]) * x[:, d:] with the tanh form of gelu."""
    d = x.shape[-1] // 2
    a = x[..., :d].float()
    return (torch.nn.functional.gelu(a, approximate="tanh") *
            x[..., d:].float()).to(x.dtype)


def sigmoid_group_topk(logits, correction, topk, n_group, keep, scale):
    """Sigmoid routing with group limits: s = sigmoid(logits); the
    choice runs on s + correction among the experts of the ``keep``
    groups (of ``n_group`` equal neighbour groups) whose two best choice
    scores sum highest, everything else counting as -inf; the weights
    are the chosen s over their sum (+ 1e-20), times ``scale``.
    n_group <= 1: no group limit. Ties go to the lower index."""
    T, E = logits.shape
    s = torch.sigmoid(logits.float())
    sel = s + correction.float() if correction is not None else s.clone()
    if n_group > 1:
        per = E // n_group
        g = sel.view(T, n_group, per)
        gscore = g.topk(min(2, per), dim=-1)[0].sum(-1)
        order = torch.sort(gscore, dim=-1, descending=True, stable=True)[1]
        mask = torch.zeros(T, n_group, dtype=torch.bool)
        mask.scatter_(1, order[:, :keep], True)
        mask = mask.unsqueeze(-1).expand(T, n_group, per).reshape(T, E)
        sel = sel.masked_fill(~mask, float("-inf"))
    ids = torch.sort(sel, dim=-1, descending=True, stable=True)[1][:, :topk]
    w = s.gather(1, ids)
    w = w / (w.sum(-1, keepdim=True) + 1e-20) * scale
    return w, ids.to(torch.int32)


def qk_norm_rope_store(q, k, v, q_w, k_w, positions, slot_mapping, freqs,
                       mag, rot_dims, k_cache, v_cache, H, G, D, Dv, eps,
                       half_layout=False, norm_last=False, do_norm=True,
                       v_freqs=None, norm_span=False, v_unit=False,
                       q_out=None):
    """Per-head RMS norm (plain weight, or none when the weight is None)
    + rotary on q (in place) and k; k, v land in the paged cache rows
    ``slot_mapping``. ``k`` None: a layer that reads another layer's
    cache. ``half_layout``: dimension i pairs with i + rot_dims/2
    instead of (2i, 2i+1); ``norm_last``: rotate first, then norm;
    ``do_norm`` False: rotary only. ``v_freqs`` [Dv/2]: every value row
    is turned by its own position over all of Dv before it is stored.
    ``norm_span``: the RMS is taken over all heads of a token's row at
    once and the weights cover the row ([heads * D]). ``v_unit``: every
    value head is brought to unit RMS (eps, no weight) before the
    store."""
    T = q.shape[0]
    ang = positions[:T].double()[:, None] * freqs.double()[None, :rot_dims // 2]
    cos = (torch.cos(ang).float() * mag)[:, None, :]
    sin = (torch.sin(ang).float() * mag)[:, None, :]
    half = rot_dims // 2

    def norm(xf, w):
        if not do_norm:
            return xf
        if norm_span:
            ms = (xf * xf).mean((-2, -1), keepdim=True)
            xf = xf * torch.rsqrt(ms + eps)
            return xf if w is None else xf * w.float().view(xf.shape[1:])
        xf = xf * torch.rsqrt((xf * xf).mean(-1, keepdim=True) + eps)
        return xf if w is None else xf * w.float()

    def rotate(xf):
        if half_layout:
            a, b = xf[..., :half], xf[..., half:rot_dims]
            return torch.cat([a * cos - b * sin, b * cos + a * sin,
                              xf[..., rot_dims:]], dim=-1)
        a, b = xf[..., 0:rot_dims:2], xf[..., 1:rot_dims:2]
        rot = torch.stack([a * cos - b * sin, b * cos + a * sin], dim=-1)
        return torch.cat([rot.flatten(-2), xf[..., rot_dims:]], dim=-1)

    def prep(x, w, heads):
        xf = x.float().reshape(T, heads, D)
        if norm_last:
            return norm(rotate(xf), w)
        return rotate(norm(xf, w))

    (q if q_out is None else q_out).copy_(
        prep(q, q_w, H).reshape(T, H * D).to(q.dtype))
    if k is None:
        return
    rows = slot_mapping[:T]
    kc = k_cache.view(-1, G, D)
    vc = v_cache.view(-1, G, Dv)
    kc[rows] = prep(k, k_w, G).to(k_cache.dtype)
    vv = v.reshape(T, G, Dv)
    if v_unit:
        vf = vv.float()
        vv = vf * torch.rsqrt((vf * vf).mean(-1, keepdim=True) + eps)
    if v_freqs is not None:
        vv = rotate_scale_rows(vv.reshape(T, G * Dv), positions, v_freqs,
                               G, Dv, 1.0, 1.0, half_layout
                               ).reshape(T, G, Dv)
    vc[rows] = vv.to(v_cache.dtype)


def rotate_scale_rows(x, positions, freqs, heads, D, sign, scale,
                      half_layout=False, out=None):
    """Every head row of x [T, heads*D]: pairs (2m, 2m+1) (half
    layout: (m, m + D/2)) turned by sign * position * freqs[m], then
    scaled. ``out`` may be a column block of a wider buffer."""
    T = x.shape[0]
    half = D // 2
    ang = positions[:T].double()[:, None] * freqs.double()[None, :half]
    cos = torch.cos(ang).float()[:, None, :]
    sin = torch.sin(ang).float()[:, None, :] * sign
    xf = x.float().reshape(T, heads, D)
    if half_layout:
        a, b = xf[..., :half], xf[..., half:]
        res = torch.cat([a * cos - b * sin, b * cos + a * sin], dim=-1)
    else:
        a, b = xf[..., 0::2], xf[..., 1::2]
        res = torch.stack([a * cos - b * sin, b * cos + a * sin],
                          dim=-1).flatten(-2)
    res = (res * scale).reshape(T, heads * D).to(x.dtype)
    if out is None:
        return res
    out.copy_(res)
    return out


def rms_weight_store(x, w, eps, cache=None, slot_mapping=None):
    """Weighted RMS norm of rows (fp32 inside, result in x's dtype);
    with ``cache`` [pages, page, 1, n] the rows also land in their paged
    slots."""
    xf = x.float()
    y = (xf * torch.rsqrt((xf * xf).mean(-1, keepdim=True) + eps)
         * w.float()).to(x.dtype)
    if cache is not None:
        cache.view(-1, x.shape[1])[slot_mapping[:x.shape[0]]] = \
            y.to(cache.dtype)
    return y


def hyper_streams(xs, y=None, y2=None, gate=None, mix=None, out_w=None,
                  read=None, dtype=None):
    """Multi-stream residual xs [S, T, W] fp32. With ``y``: every
    stream is rewritten from the old ones, x_t = sum_s mix[s, t] x_s +
    out_w[t] * (y + sigmoid(gate) * y2) (in place). With ``read`` =
    (in_w [S], gain [1], eps): returns gain * u / rms(u) in ``dtype``,
    u = sum_s in_w[s] x_s of the (updated) streams."""
    if y is not None:
        yv = y.float()
        if y2 is not None:
            g = torch.sigmoid(gate.float()) if gate is not None else 1.0
            yv = yv + g * y2.float()
        new = torch.einsum("st,snw->tnw", mix.float(), xs) \
            + out_w.float()[:, None, None] * yv[None]
        xs.copy_(new)
    if read is None:
        return None
    in_w, gain, eps = read
    u = torch.einsum("s,snw->nw", in_w.float(), xs)
    h = u * torch.rsqrt((u * u).mean(-1, keepdim=True) + eps) * gain.float()
    return h.to(dtype)


def mingru_varlen(zx, gp, state, slots, has_init, query_start_loc, scale,
                  out=None):
    """Ragged minGRU: zx [T, 2C] = update-gate | candidate
    pre-activations, gp [T, C] read-out gate; S_t = (1 - z) S_{t-1} +
    z c with z = sigmoid(zp), c = up + 1/2 (up >= 0) or sigmoid(up);
    out_t = scale * S_t * silu(gp_t). state [slots, C] fp32 in place."""
    T, C = gp.shape
    res = torch.empty(T, C, dtype=torch.float32)
    qsl = query_start_loc.tolist()
    z = torch.sigmoid(zx[:, :C].float())
    up = zx[:, C:].float()
    cand = torch.where(up >= 0, up + 0.5, torch.sigmoid(up))
    g = gp.float()
    g = g * torch.sigmoid(g)
    st = state.view(-1, C)
    for b in range(len(qsl) - 1):
        slot = int(slots[b])
        S = st[slot].clone() if int(has_init[b]) else torch.zeros(C)
        for t in range(qsl[b], qsl[b + 1]):
            S = (1 - z[t]) * S + z[t] * cand[t]
            res[t] = scale * S * g[t]
        if qsl[b + 1] > qsl[b]:
            st[slot] = S
    res = res.to(zx.dtype)
    if out is None:
        return res
    out.copy_(res)
    return out


def clamp_swiglu(x, limit, alpha):
    """x [rows, 2d] = gate | up: min(g, limit) * sigmoid(alpha g) *
    (clamp(u, -limit, limit) + 1)."""
    d = x.shape[-1] // 2
    g = x[..., :d].float().clamp(max=limit)
    u = x[..., d:].float().clamp(-limit, limit)
    return (g * torch.sigmoid(alpha * g) * (u + 1)).to(x.dtype)


def window_attention(q, gate, k_cache, v_cache, block_table, seq_lens,
                     query_start_loc, scale, window, keep_first, sink,
                     sinks=None, softcap=0.0):
    """Ragged paged attention: position i sees j <= i with i - j < window
    (window <= 0: all) or j < keep_first; ``sink`` adds 1 to the softmax
    denominator, ``sinks`` [H] adds exp(sinks[h]) instead; ``softcap``:
    scores become cap * tanh(score / cap); ``gate`` multiplies the heads
    by sigmoid(gate)."""
    page, G, D = k_cache.shape[1:]
    Dv = v_cache.shape[3]
    T = q.shape[0]
    H = q.shape[1] // D
    out = torch.zeros(T, H, Dv, dtype=torch.float32)
    qsl = query_start_loc.tolist()
    lens = seq_lens.tolist()
    qf = q.float().reshape(T, H, D)
    for b in range(len(lens)):
        s, e, L = qsl[b], qsl[b + 1], lens[b]
        if e == s:
            continue
        pages = block_table[b, :-(-L // page)].long()
        kk = k_cache[pages].reshape(-1, G, D)[:L].float()
        vv = v_cache[pages].reshape(-1, G, Dv)[:L].float()
        pos_i = torch.arange(L - (e - s), L)[:, None]
        pos_j = torch.arange(L)[None, :]
        see = pos_j <= pos_i
        if window > 0:
            see = see & ((pos_i - pos_j < window) | (pos_j < keep_first))
        kk = kk.repeat_interleave(H // G, dim=1)
        vv = vv.repeat_interleave(H // G, dim=1)
        sc = torch.einsum("ihd,jhd->hij", qf[s:e], kk) * scale
        if softcap:
            sc = softcap * torch.tanh(sc / softcap)
        sc = sc.masked_fill(~see[None], float("-inf"))
        m = sc.amax(-1, keepdim=True)
        if sinks is not None:
            sk = sinks.float().reshape(H, 1, 1)
        elif sink:
            sk = torch.zeros(H, 1, 1)
        else:
            sk = None
        if sk is not None:
            m = torch.maximum(m, sk)
        p = torch.exp(sc - m)
        den = p.sum(-1, keepdim=True)
        if sk is not None:
            den = den + torch.exp(sk - m)
        out[s:e] = torch.einsum("hij,jhd->ihd", p / den, vv)
    out = out.reshape(T, H * Dv)
    if gate is not None:
        out = out * torch.sigmoid(gate.float())
    return out.to(q.dtype)


def talking_attention(q, k_cache, v_cache, block_table, seq_lens,
                      query_start_loc, scale, talk, sink):
    """Ragged paged causal attention whose per-head score planes are
    mixed across heads before the softmax: s'_h = sum_g talk[h, g] s_g
    with s_g = scale * q_g . k. ``sink`` [H] (or None) adds exp(sink_h)
    to head h's softmax denominator. Scores and weights are fp32."""
    page, G, D = k_cache.shape[1:]
    Dv = v_cache.shape[3]
    T = q.shape[0]
    H = q.shape[1] // D
    out = torch.zeros(T, H, Dv, dtype=torch.float32)
    qsl = query_start_loc.tolist()
    lens = seq_lens.tolist()
    qf = q.float().reshape(T, H, D)
    mix = talk.float()
    for b in range(len(lens)):
        s, e, L = qsl[b], qsl[b + 1], lens[b]
        if e == s:
            continue
        pages = block_table[b, :-(-L // page)].long()
        kk = k_cache[pages].reshape(-1, G, D)[:L].float()
        vv = v_cache[pages].reshape(-1, G, Dv)[:L].float()
        pos_i = torch.arange(L - (e - s), L)[:, None]
        see = torch.arange(L)[None, :] <= pos_i
        kk = kk.repeat_interleave(H // G, dim=1)
        vv = vv.repeat_interleave(H // G, dim=1)
        sc = torch.einsum("ihd,jhd->hij", qf[s:e], kk) * scale
        sc = torch.einsum("hg,gij->hij", mix, sc)
        sc = sc.masked_fill(~see[None], float("-inf"))
        m = sc.amax(-1, keepdim=True)
        if sink is not None:
            sk = sink.float().view(H, 1, 1)
            m = torch.maximum(m, sk)
        p = torch.exp(sc - m)
        den = p.sum(-1, keepdim=True)
        if sink is not None:
            den = den + torch.exp(sk - m)
        out[s:e] = torch.einsum("hij,jhd->ihd", p / den, vv)
    return out.reshape(T, H * Dv).to(q.dtype)


def xielu(x: torch.Tensor, a_pos: float, a_neg: float) -> torch.Tensor:
    """z > 0: a_pos z^2 + z/2; z <= 0: a_neg (exp(z) - 1 - z) + z/2."""
    z = x.float()
    neg = a_neg * (torch.expm1(z.clamp(max=0.0)) - z) + 0.5 * z
    return torch.where(z > 0, a_pos * z * z + 0.5 * z, neg).to(x.dtype)


def relu2(x: torch.Tensor) -> torch.Tensor:
    r = torch.relu(x.float())
    return (r * r).to(x.dtype)


def topk_then_softmax(logits: torch.Tensor, topk: int):
    """MoE routing that picks the ``topk`` largest LOGITS and softmaxes
    over the chosen ones only. Returns (weights fp32 [T,K], ids [T,K])."""
    vals, ids = torch.topk(logits.float(), topk, dim=-1)
    return torch.softmax(vals, dim=-1), ids.to(torch.int32)
