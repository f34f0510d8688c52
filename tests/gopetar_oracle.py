"""Plain float64 implementation of the Gopetar decoder, one function
per mechanism, written from the design's equations. It is the oracle
the engine tests compare against and shares no code with the product
path: whole sequences, dense masks, python loops over time, no cache.

A model is (config dict, {tensor name: tensor}); names follow the
checkpoint layout (``l<i>.mix.left.q`` ...).
"""

import math

import torch

F64 = torch.float64


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def scalar_norm(x, g, eps):
    """RMS norm whose gain is one number for all coordinates."""
    return rms(x, eps) * g


def weight_norm(x, w, eps):
    return rms(x, eps) * w


# ---------------------------------------------------------------- rotary
def pair_freqs(dims, base):
    i = torch.arange(dims // 2, dtype=F64)
    return base ** (-2.0 * i / dims)


def scaled_freqs(f, sc):
    """Wavelength-dependent slow-down: short waves keep f, long waves
    run at f / factor, a linear blend in between."""
    if not sc:
        return f
    factor, low, high = float(sc["factor"]), float(sc["low"]), \
        float(sc["high"])
    orig = float(sc["original"])
    out = f.clone()
    for n in range(f.numel()):
        wl = 2 * math.pi / float(f[n])
        if wl < orig / high:
            continue
        if wl > orig / low:
            out[n] = f[n] / factor
        else:
            s = (orig / wl - low) / (high - low)
            out[n] = (1 - s) * f[n] / factor + s * f[n]
    return out


def rotate_pairs(x, pos, f, sign=1.0):
    """x [T, heads, D]; dims (2m, 2m+1), m < len(f), turn by
    sign * pos * f[m]; the remaining dims pass through."""
    n = f.numel()
    ang = sign * pos.to(F64)[:, None] * f[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    a, b = x[..., 0:2 * n:2], x[..., 1:2 * n:2]
    out = x.clone()
    out[..., 0:2 * n:2] = a * c - b * s
    out[..., 1:2 * n:2] = b * c + a * s
    return out


# ---------------------------------------------------------------- mixers
def window_sink_attention(h, W, p, m):
    """The left branch: GQA, biased projections, partial scaled rotary
    on q/k, values rotated by their own position over all vdim and the
    head sums rotated back by the query position, tanh-capped scores, a
    sliding window and a per-head sink in the softmax denominator."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q = (h @ W[p + "q"].T + W[p + "q.b"]).reshape(T, H, D)
    k = (h @ W[p + "k"].T + W[p + "k.b"]).reshape(T, G, D)
    v = (h @ W[p + "v"].T + W[p + "v.b"]).reshape(T, G, Dv)
    rot = m.get("rot")
    fv = None
    if rot:
        if rot.get("dims"):
            f = scaled_freqs(pair_freqs(rot["dims"], rot["base"]),
                             rot.get("scaling"))
            q, k = rotate_pairs(q, pos, f), rotate_pairs(k, pos, f)
        # the values turn over all of vdim whatever part of q/k does
        fv = pair_freqs(Dv, rot["base"])
        v = rotate_pairs(v, pos, fv)
    out = torch.zeros(T, H, Dv, dtype=F64)
    cap = m.get("softcap")
    win = m["mask"]["size"] if m.get("mask") else 0
    for hh in range(H):
        g = hh // (H // G)
        s = (q[:, hh] @ k[:, g].T) * m["scale"]
        if cap:
            s = cap * torch.tanh(s / cap)
        i, j = pos[:, None], pos[None, :]
        see = (j <= i)
        if win:
            see = see & (i - j < win)
        s = s.masked_fill(~see, float("-inf"))
        e = torch.exp(s)
        den = e.sum(-1, keepdim=True) + torch.exp(W[p + "sink"][hh])
        out[:, hh] = (e / den) @ v[:, g]
    if fv is not None:
        out = rotate_pairs(out, pos, fv, sign=-1.0)
    return out.reshape(T, H * Dv) @ W[p + "o"].T


def min_gru(h, W, p, state=None):
    """The right branch: S_t = (1 - z_t) S_{t-1} + z_t c_t, gates from
    the current token only; read-out W_o (S_t * silu(W_g h_t))."""
    T = h.shape[0]
    z = torch.sigmoid(h @ W[p + "z"].T + W[p + "z.b"])
    u = h @ W[p + "x"].T + W[p + "x.b"]
    cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    gate = h @ W[p + "g"].T
    S = torch.zeros(z.shape[1], dtype=F64) if state is None else state
    rows = []
    for t in range(T):
        S = (1 - z[t]) * S + z[t] * cand[t]
        rows.append(S * gate[t] * torch.sigmoid(gate[t]))
    return torch.stack(rows) @ W[p + "o"].T


def parallel_mixer(h, W, p, m):
    left = window_sink_attention(h, W, p + "left.", m["left"])
    right = min_gru(h, W, p + "right.")
    return m["left_scale"] * left + m["right_scale"] * right


def latent_of(h, W, p, eps):
    return weight_norm(h @ W[p + "dkv"].T, W[p + "dkv.norm"], eps)


def latent_attention(h, W, p, m, eps, latent):
    """Causal attention without positions whose keys and values are
    up-projections of a normed low-rank latent (``latent`` [T, rank],
    this layer's own or another layer's); queries go through a normed
    latent of their own."""
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    cq = weight_norm(h @ W[p + "dq"].T, W[p + "dq.norm"], eps)
    q = (cq @ W[p + "uq"].T).reshape(T, H, D)
    k = (latent @ W[p + "uk"].T).reshape(T, H, D)
    v = (latent @ W[p + "uv"].T).reshape(T, H, Dv)
    pos = torch.arange(T)
    see = pos[None, :] <= pos[:, None]
    out = torch.zeros(T, H, Dv, dtype=F64)
    for hh in range(H):
        s = (q[:, hh] @ k[:, hh].T) * m["scale"]
        s = s.masked_fill(~see, float("-inf"))
        out[:, hh] = torch.softmax(s, -1) @ v[:, hh]
    return out.reshape(T, H * Dv) @ W[p + "o"].T


# ---------------------------------------------------------------- ff
def clamped_expert(h, W, p, limit):
    g = torch.clamp(h @ W[p + "gate"].T, max=limit)
    u = torch.clamp(h @ W[p + "up"].T, -limit, limit)
    y = g * torch.sigmoid(1.702 * g) * (u + 1)
    return y @ W[p + "down"].T


def moe(h, W, p, mlp):
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    logits = h @ W[p + "router"].T
    vals, ids = torch.topk(logits, top, dim=-1)
    wts = torch.softmax(vals, -1)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for n in range(top):
            e = int(ids[t, n])
            out[t] += wts[t, n] * clamped_expert(
                h[t:t + 1], W, p + "e%d." % e, mlp["expert"]["limit"])[0]
    sh = mlp.get("shared")
    if sh:
        gate = torch.sigmoid(h @ W[p + "shared.sg"].T)
        out = out + gate * clamped_expert(h, W, p + "shared.", sh["limit"])
    return out


# ---------------------------------------------------------------- model
def forward(cfg, W, tokens, probe=None):
    """Logits [T, vocab] of one whole sequence. ``probe(i, x)`` gets the
    summed stream after every layer."""
    W = {k: v.to(F64) for k, v in W.items()}
    eps = cfg["norm"]["eps"]
    S = int(cfg.get("streams", 1) or 1)
    x0 = W["embed"][torch.as_tensor(tokens)] * cfg["embedding"]["scale"]
    xs = [x0.clone() for _ in range(S)]
    latents = {}

    def sublayer(q, i, fn):
        nonlocal xs
        pre = "l%d." % i
        g = W[pre + "norm%d" % q]
        if S == 1 and (pre + "hc%d.in" % q) not in W:
            xs = [xs[0] + fn(scalar_norm(xs[0], g, eps))]
            return
        hin, hout = W[pre + "hc%d.in" % q], W[pre + "hc%d.out" % q]
        mix = W[pre + "hc%d.mix" % q]
        u = sum(hin[s] * xs[s] for s in range(S))
        y = fn(scalar_norm(u, g, eps))
        xs = [sum(mix[s, t] * xs[s] for s in range(S)) + hout[t] * y
              for t in range(S)]

    for i, layer in enumerate(cfg["layers"]):
        p = "l%d.mix." % i
        m = layer["mixer"]
        if layer["type"] == "parallel":
            sublayer(1, i, lambda h: parallel_mixer(h, W, p, m))
        elif layer["type"] == "latent_attention":
            def mixer(h):
                src = m.get("kv_from")
                if src is None:
                    latents[i] = latent_of(h, W, p, eps)
                    src = i
                return latent_attention(h, W, p, m, eps, latents[src])
            sublayer(1, i, mixer)
        else:
            raise ValueError(layer["type"])
        if layer.get("mlp"):
            sublayer(2, i, lambda h: moe(h, W, "l%d.mlp." % i,
                                         layer["mlp"]))
        if probe is not None:
            probe(i, sum(xs))
    x = scalar_norm(sum(xs), W["final.norm"], eps)
    return x @ W["head"].T
