"""A plain, slow Sofunex in float64, one function per mechanism.

Written from the design's equations only; shares no code with
gllm_amd. ``forward`` runs one whole sequence from position 0 and
returns the logits of every position (and, on request, the residual
stream after every layer run).

cfg: the parsed config.json (a dict); W: name -> float64 tensor.
"""

import math

import torch

F64 = torch.float64


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(
        math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def token_shift(h, mu):
    """h [T, W]: every row moves towards the row before it (zeros ahead
    of the first) by the per-channel amount mu."""
    prev = torch.zeros_like(h)
    prev[1:] = h[:-1]
    return h + (prev - h) * mu


def short_conv(u, w):
    """u [T, C], w [C, taps]; the last tap sits on the current token."""
    T, C = u.shape
    taps = w.shape[1]
    y = torch.zeros_like(u)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += w[:, j] * u[s]
    return y


def rotate_half(x, dims, base, factor):
    """x [T, H, D]; the first ``dims`` dims of a head turn, dim i with
    dim i + dims/2, by position * base^(-2i/dims) / factor."""
    if not dims:
        return x
    T = x.shape[0]
    half = dims // 2
    i = torch.arange(half, dtype=F64)
    f = base ** (-2.0 * i / dims) / factor
    ang = torch.arange(T, dtype=F64)[:, None] * f[None, :]
    c, s = ang.cos()[:, None, :], ang.sin()[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    out = x.clone()
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


def window_attention(q, k, v, scale, window):
    """q [T, H, D], k [T, G, D], v [T, G, Dv]; position i sees j with
    0 <= i - j < window (window None: every j <= i)."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    for h in range(H):
        g = h // (H // G)
        for i in range(T):
            lo = 0 if not window else max(0, i - window + 1)
            s = (k[lo:i + 1, g] @ q[i, h]) * scale
            p = torch.softmax(s, 0)
            out[i, h] = p @ v[lo:i + 1, g]
    return out


def left_branch(h, m, W, pre, eps):
    H, G = m["heads"], m["kv_heads"]
    D, Dv = m["dim"], m["vdim"]
    T = h.shape[0]

    def proj(name):
        y = h @ W[pre + name].T
        if pre + name + ".b" in W:
            y = y + W[pre + name + ".b"]
        if pre + name + ".conv" in W:
            y = short_conv(y, W[pre + name + ".conv"])
        return y

    q, k, v = proj("q"), proj("k"), proj("v")
    q = unit_rms(q, eps) * W[pre + "q.norm"]
    k = unit_rms(k, eps) * W[pre + "k.norm"]
    rot = m.get("rot") or {}
    dims = int(rot.get("dims", 0) or 0)
    factor = float((rot.get("scaling") or {}).get("factor", 1.0))
    q = rotate_half(q.view(T, H, D), dims, float(rot.get("base", 1.0)),
                    factor)
    k = rotate_half(k.view(T, G, D), dims, float(rot.get("base", 1.0)),
                    factor)
    v = unit_rms(v.view(T, G, Dv), eps)
    window = (m.get("mask") or {}).get("size")
    o = window_attention(q, k, v, float(m["scale"]), window)
    y = o.reshape(T, H * Dv) @ W[pre + "o"].T
    if pre + "o.b" in W:
        y = y + W[pre + "o.b"]
    return y


def delta_recurrence(r, k, v, w, a):
    """All [T, H, D]. S [D(key), D(value)] per head, from zero:
    S <- diag(w) S - (a u)(u^T S) + k v^T with u = k / |k|; o = S^T r."""
    T, H, D = r.shape
    o = torch.zeros(T, H, D, dtype=F64)
    for h in range(H):
        S = torch.zeros(D, D, dtype=F64)
        for t in range(T):
            u = k[t, h] / torch.sqrt((k[t, h] ** 2).sum() + 1e-6)
            S = w[t, h][:, None] * S \
                - torch.outer(a[t, h] * u, u @ S) \
                + torch.outer(k[t, h], v[t, h])
            o[t, h] = S.T @ r[t, h]
    return o


def right_branch(h, m, W, pre, eps):
    H, D = m["heads"], m["dim"]
    T = h.shape[0]
    r = (h @ W[pre + "r"].T).view(T, H, D)
    k = (h @ W[pre + "k"].T).view(T, H, D)
    v = (h @ W[pre + "v"].T).view(T, H, D)
    lw = torch.tanh(h @ W[pre + "w1"].T) @ W[pre + "w2"].T + W[pre + "w0"]
    w = torch.exp(-math.exp(-0.5) * torch.sigmoid(lw)).view(T, H, D)
    a = torch.sigmoid(h @ W[pre + "a"].T + W[pre + "a.b"]).view(T, H, D)
    o = delta_recurrence(r, k, v, w, a)
    o = unit_rms(o, eps).reshape(T, H * D) * W[pre + "norm"]
    o = o * torch.sigmoid(h @ W[pre + "g"].T)
    return o @ W[pre + "o"].T


def parallel_mixer(h, m, W, pre, eps):
    return float(m.get("left_scale", 1.0)) * left_branch(
        h, m["left"], W, pre + "left.", eps) \
        + float(m.get("right_scale", 1.0)) * right_branch(
            h, m["right"], W, pre + "right.", eps)


def glu(h, W, pre, act):
    return (act(h @ W[pre + "gate"].T) * (h @ W[pre + "up"].T)) \
        @ W[pre + "down"].T


def route(h, mlp, W, pre):
    """Returns per token the chosen experts and their weights."""
    r = mlp["router"]
    E, top = r["experts"], r["top"]
    s = torch.sigmoid(h @ W[pre + "router"].T)
    choice = s.clone()
    if pre + "correction" in W:
        choice = choice + W[pre + "correction"]
    groups = r.get("groups")
    if groups:
        n, keep = groups["count"], groups["keep"]
        per = E // n
        for t in range(h.shape[0]):
            gs = [choice[t, g * per:(g + 1) * per].topk(min(2, per))[0].sum()
                  for g in range(n)]
            best = sorted(range(n), key=lambda g: (-float(gs[g]), g))[:keep]
            for g in range(n):
                if g not in best:
                    choice[t, g * per:(g + 1) * per] = -math.inf
    ids = choice.topk(top, dim=-1)[1]
    wts = s.gather(1, ids)
    wts = wts / (wts.sum(-1, keepdim=True) + 1e-20) * float(
        r.get("scale", 1.0))
    return ids, wts


def moe(h, mlp, W, pre):
    ids, wts = route(h, mlp, W, pre)
    y = torch.zeros(h.shape[0], W[pre + "e0.down"].shape[0], dtype=F64)
    for t in range(h.shape[0]):
        for j in range(ids.shape[1]):
            e = int(ids[t, j])
            y[t] += wts[t, j] * glu(h[t:t + 1], W, f"{pre}e{e}.", silu)[0]
    if mlp.get("shared"):
        y = y + glu(h, W, pre + "shared.", silu)
    return y


def feed_forward(h, mlp, W, pre):
    if mlp["kind"] == "dense":
        return glu(h, W, pre, gelu_tanh)
    return moe(h, mlp, W, pre)


def layer_run(x, i, cfg, W):
    lay = cfg["layers"][i]
    eps = float(cfg["norm"]["eps"])
    m = float(cfg.get("residual_mult", 1.0))
    p = f"l{i}."
    assert lay["type"] == "parallel"
    h = unit_rms(x, eps) * W[p + "norm1"]
    if p + "shift" in W:
        h = token_shift(h, W[p + "shift"])
    y = parallel_mixer(h, lay["mixer"], W, p + "mix.", eps)
    x = x + m * (unit_rms(y, eps) * W[p + "norm1b"])
    if lay.get("mlp"):
        h = unit_rms(x, eps) * W[p + "norm2"]
        y = feed_forward(h, lay["mlp"], W, p + "mlp.")
        x = x + m * (unit_rms(y, eps) * W[p + "norm2b"])
    return x


def run_order(cfg):
    """[(layer, pass number or None when the layer opens no pass)]."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    a, b, times = loop["start"], loop["stop"], loop["times"]
    order = [(i, None) for i in range(a)]
    for t in range(times):
        order += [(i, t if i == a else None) for i in range(a, b)]
    return order + [(i, None) for i in range(b, n)]


def forward(cfg, W, tokens, probe=None):
    eps = float(cfg["norm"]["eps"])
    x = W["embed"][torch.as_tensor(tokens)] * float(
        (cfg.get("embedding") or {}).get("scale", 1.0))
    for i, opens in run_order(cfg):
        if opens is not None:
            x = x + W["loop.step"][opens]
        x = layer_run(x, i, cfg, W)
        if probe is not None:
            probe.append(x.clone())
    x = unit_rms(x, eps) * W["final.norm"]
    return x @ W["head"].T
