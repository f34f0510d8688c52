"""Gopetar decoder: the engine (scheduler, paged KV pool, state pool,
batch builder, ops) against the plain float64 oracle in
gopetar_oracle.py.

Every test builds its own small configuration and random bf16 weights,
replays token schedules through the product's trace-replay entry point
(or LLM.generate) and compares logits with the oracle run on each whole
sequence alone. CPU runs exercise the engine with the torch reference
ops; the same tests marked ``gpu`` exercise the HIP kernels in fp32
(tight tolerance) and bf16.
"""

import json
import math
import os
import tempfile

import numpy as np
import pytest
import torch

import gopetar_oracle as oracle

DEVICES = [pytest.param("cpu", "float32", id="cpu-f32"),
           pytest.param("cuda", "float32", id="gpu-f32",
                        marks=pytest.mark.gpu),
           pytest.param("cuda", "bfloat16", id="gpu-bf16",
                        marks=pytest.mark.gpu)]
TOL = {"float32": 3e-4, "bfloat16": 8e-2}


# ------------------------------------------------------------------ models
def moe_ff(experts=6, top=2, ff=16, limit=1.2, shared=24, shared_limit=2.5):
    mlp = {"kind": "moe", "expert": {"ff": ff, "limit": limit},
           "router": {"experts": experts, "top": top}}
    if shared:
        mlp["shared"] = {"ff": shared, "limit": shared_limit}
    return mlp


def parallel(heads=4, kv_heads=2, dim=16, vdim=12, window=9, rot_dims=8,
             base=10000.0, scaling=None, scale=0.3, softcap=5.0, gru=20,
             left_scale=0.7, right_scale=1.3, mlp=None):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
            "mask": {"size": window}, "scale": scale, "softcap": softcap}
    if rot_dims is not None:
        left["rot"] = {"dims": rot_dims, "base": base}
        if scaling:
            left["rot"]["scaling"] = scaling
    return {"type": "parallel", "mlp": mlp,
            "mixer": {"left": left, "left_scale": left_scale,
                      "right": {"width": gru}, "right_scale": right_scale}}


def latent(heads=3, dim=8, vdim=10, kv_rank=12, q_rank=14, scale=0.4,
           kv_from=None, mlp=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": kv_rank,
         "q_rank": q_rank, "scale": scale}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


# wavelengths 2 pi / f of base 100 over 8 dims: 6.3, 20, 63, 199; with
# original/high = 12 and original/low = 48 the first pair keeps its
# frequency, the second is blended, the last two are slowed
SCALING = {"factor": 4.0, "low": 2.0, "high": 8.0, "original": 96}


def make_config(layers, width=32, vocab=70, eps=1e-5, streams=2,
                embed_scale=3.0):
    return {"architecture": "Gopetar", "embedding": {"scale": embed_scale},
            "layers": layers, "norm": {"eps": eps}, "streams": streams,
            "vocab": vocab, "width": width}


def make_weights(cfg, seed, hc=True):
    g = torch.Generator().manual_seed(seed)
    W, S = cfg["width"], cfg["streams"]
    w = {}

    def lin(name, out, inp, gain=1.0):
        w[name] = torch.randn(out, inp, generator=g) * gain / inp ** 0.5

    def vec(name, n, gain=0.5):
        w[name] = gain * torch.randn(n, generator=g)

    w["embed"] = torch.randn(cfg["vocab"], W, generator=g) / 3.0
    w["final.norm"] = 1.0 + 0.2 * torch.randn((), generator=g)
    lin("head", cfg["vocab"], W)
    for i, layer in enumerate(cfg["layers"]):
        p = "l%d." % i
        m = layer["mixer"]
        for q in (1, 2):
            if q == 2 and not layer.get("mlp"):
                continue
            w[p + "norm%d" % q] = 1.0 + 0.2 * torch.randn((), generator=g)
            if hc:
                w[p + "hc%d.in" % q] = torch.full((S,), 1.0 / S) \
                    + 0.3 * torch.randn(S, generator=g)
                w[p + "hc%d.out" % q] = 1.0 + 0.3 * torch.randn(S,
                                                                generator=g)
                w[p + "hc%d.mix" % q] = torch.eye(S) \
                    + 0.3 * torch.randn(S, S, generator=g)
        if layer["type"] == "parallel":
            a = m["left"]
            H, G, D, Dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            C = m["right"]["width"]
            lin(p + "mix.left.q", H * D, W, 2.0)
            lin(p + "mix.left.k", G * D, W, 2.0)
            lin(p + "mix.left.v", G * Dv, W)
            vec(p + "mix.left.q.b", H * D)
            vec(p + "mix.left.k.b", G * D)
            vec(p + "mix.left.v.b", G * Dv)
            vec(p + "mix.left.sink", H, 1.0)
            lin(p + "mix.left.o", W, H * Dv)
            lin(p + "mix.right.z", C, W, 2.0)
            lin(p + "mix.right.x", C, W, 2.0)
            vec(p + "mix.right.z.b", C)
            vec(p + "mix.right.x.b", C)
            lin(p + "mix.right.g", C, W, 2.0)
            lin(p + "mix.right.o", W, C)
        else:
            H, D, Dv = m["heads"], m["dim"], m["vdim"]
            R, Q = m["kv_rank"], m["q_rank"]
            lin(p + "mix.dq", Q, W)
            w[p + "mix.dq.norm"] = 1.0 + 0.2 * torch.randn(Q, generator=g)
            lin(p + "mix.uq", H * D, Q, 2.0)
            if m.get("kv_from") is None:
                lin(p + "mix.dkv", R, W)
                w[p + "mix.dkv.norm"] = 1.0 + 0.2 * torch.randn(R,
                                                                generator=g)
            lin(p + "mix.uk", H * D, R, 2.0)
            lin(p + "mix.uv", H * Dv, R)
            lin(p + "mix.o", W, H * Dv)
        mlp = layer.get("mlp")
        if not mlp:
            continue
        E, ff = mlp["router"]["experts"], mlp["expert"]["ff"]
        lin(p + "mlp.router", E, W, 2.0)
        for e in range(E):
            lin(p + "mlp.e%d.gate" % e, ff, W, 2.0)
            lin(p + "mlp.e%d.up" % e, ff, W, 2.0)
            lin(p + "mlp.e%d.down" % e, W, ff)
        if mlp.get("shared"):
            fs = mlp["shared"]["ff"]
            lin(p + "mlp.shared.gate", fs, W, 2.0)
            lin(p + "mlp.shared.up", fs, W, 2.0)
            lin(p + "mlp.shared.down", W, fs)
            lin(p + "mlp.shared.sg", 1, W, 2.0)
    return {k: v.to(torch.bfloat16).contiguous() for k, v in w.items()}


def save_model(cfg, weights):
    from safetensors.torch import save_file
    d = tempfile.mkdtemp(prefix="gopetar_test_")
    with open(os.path.join(d, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file(weights, os.path.join(d, "model.safetensors"))
    return d


# a latent layer ahead of its reader, two different parallel layers, one
# layer without a feed-forward, three streams
STACK = [latent(mlp=moe_ff()),
         parallel(mlp=moe_ff(experts=4, top=1, ff=8, shared=0),
                  scaling=SCALING, base=100.0),
         latent(heads=2, dim=12, vdim=6, q_rank=9, kv_from=0),
         parallel(heads=3, kv_heads=3, dim=10, vdim=16, window=17,
                  rot_dims=10, softcap=0, gru=13, mlp=moe_ff(top=3))]


def stack_for(dtype, layers=None):
    """fp32 runs route for real. In bf16 the 16-bit rounding of a
    router's input flips a close top-k call now and then, and here a
    flip does not stay at its position: it changes keys, latents and the
    recurrent state that every later position reads. So the multi-layer
    bf16 runs use every expert (top = experts: the grouped GEMM, the
    routing weights and their softmax still run, nothing discrete is
    left); discrete routing in bf16 is covered by the one-layer models
    of test_each_mechanism_alone, where a flip stays local."""
    layers = STACK if layers is None else layers
    if dtype != "bfloat16":
        return layers
    out = []
    for lay in layers:
        if lay.get("mlp"):
            mlp = dict(lay["mlp"])
            mlp["router"] = dict(mlp["router"],
                                 top=mlp["router"]["experts"])
            lay = dict(lay, mlp=mlp)
        out.append(lay)
    return out


# ------------------------------------------------------------------ harness
def engine(model_dir, device, dtype, max_tokens=256, slots=4, page=16):
    from gllm_amd.entrypoints.trace_replay import build_engine
    return build_engine(model_dir, dtype, max_tokens, slots, device, page)


def run_steps(llm, steps, vocab):
    """steps: [{"entries": [(rid, tokens, want)], "end": [rid]}] ->
    {rid: {position: logits}} through trace_replay.replay."""
    from gllm_amd.entrypoints.trace_replay import replay
    out = tempfile.mkdtemp(prefix="gopetar_out_")
    lines, where, at = [], [], {}
    for n, st in enumerate(steps):
        ents, rows = [], []
        for rid, toks, want in st["entries"]:
            lo = at.get(rid, 0)
            ents.append({"id": rid, "tokens": toks, "want": want})
            rows += [(rid, lo + k) for k in want]
            at[rid] = lo + len(toks)
        for rid in st.get("end", []):
            at.pop(rid, None)
        lines.append(json.dumps({"step": n, "entries": ents,
                                 "end": st.get("end", [])}))
        where.append(rows)
    replay(llm, lines, out, emit=lambda t: None)
    got = {}
    for n, rows in enumerate(where):
        if not rows:
            continue
        arr = np.fromfile(os.path.join(out, "%d.f32" % n),
                          dtype="<f4").reshape(len(rows), vocab)
        for j, (rid, pos) in enumerate(rows):
            got.setdefault(rid, {})[pos] = arr[j]
    return got


def rel_err(got, want):
    d = got.astype(np.float64) - want
    d = d - d.mean()
    c = want - want.mean()
    return float(np.sqrt((d ** 2).mean()) / np.sqrt((c ** 2).mean()))


def check_against_oracle(cfg, weights, got, prompts, tol):
    """fp32: every position within tol. bf16: the 16-bit rounding of a
    router's input can flip a close top-k call, which moves that
    position's logits by far more than rounding does; allow a few such
    positions (a wrong mechanism moves most of them)."""
    worst, refs = 0.0, {}
    for rid, rows in got.items():
        key = tuple(prompts[rid.split("#")[0]])
        if key not in refs:
            refs[key] = oracle.forward(cfg, weights, list(key)).numpy()
        errs = {pos: rel_err(lg, refs[key][pos]) for pos, lg in rows.items()}
        over = {p: e for p, e in errs.items() if not e < tol}
        if tol < 1e-2:
            assert not over, (rid, over)
        else:
            assert len(over) <= max(1, len(errs) // 16), (rid, over)
        worst = max(worst, max(errs.values()))
    return worst


def cut(rid, tokens, sizes, want_all=True):
    """One request alone, cut into portions of the given sizes."""
    steps, lo = [], 0
    for n in sizes:
        toks = tokens[lo:lo + n]
        if not toks:
            break
        steps.append({"entries": [(rid, toks, list(range(len(toks)))
                                   if want_all else [len(toks) - 1])]})
        lo += len(toks)
    assert lo == len(tokens)
    steps[-1]["end"] = [rid]
    return steps


def tokens_for(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


# ------------------------------------------------------------------ tests
MECHANISMS = {
    "parallel": ([parallel()], 2, True),
    "parallel-mha-fullrot-scaled": (
        [parallel(heads=2, kv_heads=2, dim=8, vdim=8, rot_dims=8,
                  base=100.0, scaling=SCALING, window=200)], 2, True),
    "parallel-mqa-norot-nocap": (
        [parallel(heads=3, kv_heads=1, dim=12, vdim=6, rot_dims=None,
                  softcap=0, window=1)], 3, True),
    "parallel-rot0-values-turn": (
        [parallel(rot_dims=0, vdim=20, window=5)], 1, True),
    "latent": ([latent()], 2, True),
    "latent-shared": ([latent(), latent(heads=2, dim=6, vdim=4, q_rank=5,
                                        kv_from=0)], 4, True),
    "moe": ([latent(mlp=moe_ff())], 2, True),
    "moe-all-experts-no-shared": (
        [latent(mlp=moe_ff(experts=3, top=3, ff=24, shared=0))], 2, True),
    "moe-top1-tight-limit": (
        [parallel(mlp=moe_ff(experts=5, top=1, ff=8, limit=0.3, shared=8,
                             shared_limit=0.2))], 2, True),
    "one-stream-plain-residual": ([parallel(mlp=moe_ff())], 1, False),
    # head and latent sizes that the bf16 MFMA prefill and split-KV
    # decode kernels serve (64 and 128), the latent cache as key AND
    # value operand of those kernels
    "parallel-d64-tiles": (
        [parallel(heads=4, kv_heads=2, dim=64, vdim=64, rot_dims=16,
                  window=11, scale=0.1)], 2, True),
    "parallel-d128-tiles": (
        [parallel(heads=2, kv_heads=1, dim=128, vdim=128, rot_dims=128,
                  window=40, scale=0.07, softcap=3.0)], 2, True),
    "latent-rank64-tiles": (
        [latent(heads=4, dim=16, vdim=8, kv_rank=64, q_rank=24),
         latent(heads=2, dim=8, vdim=24, kv_rank=64, q_rank=8,
                kv_from=0)], 2, True),
    "latent-rank128-tiles": (
        [latent(heads=4, dim=32, vdim=16, kv_rank=128, q_rank=40,
                scale=0.2)], 3, True),
}


@pytest.mark.parametrize("device,dtype", DEVICES)
@pytest.mark.parametrize("name", list(MECHANISMS))
@pytest.mark.parametrize("width", [32, 36], ids=["w32", "w36"])
def test_each_mechanism_alone(name, device, dtype, width):
    """Small models around one mechanism each, every position of a whole
    prompt (the first tokens included, the window passed several times).
    Width 36 is not a multiple of 8: unaligned projection rows, experts
    on the segment loop."""
    layers, streams, hc = MECHANISMS[name]
    cfg = make_config(layers, width=width, streams=streams)
    w = make_weights(cfg, 1, hc=hc)
    llm = engine(save_model(cfg, w), device, dtype)
    toks = tokens_for(cfg, 37, 2)
    # the whole prompt, then the same prompt as a portion and decoding
    # (a second request: other pages, the decode kernels)
    steps = cut("a", toks, [37]) + cut("b", toks, [30] + [1] * 7)
    got = run_steps(llm, steps, cfg["vocab"])
    check_against_oracle(cfg, w, got, {"a": toks, "b": toks}, TOL[dtype])


@pytest.mark.parametrize("device,dtype", DEVICES)
def test_layer_trail_matches(device, dtype):
    """The summed streams after every layer against the oracle's,
    through the model's layer probe."""
    cfg = make_config(stack_for(dtype), width=40, vocab=90, streams=3)
    w = make_weights(cfg, 21)
    llm = engine(save_model(cfg, w), device, dtype)
    toks = tokens_for(cfg, 19, 22)
    trail, want = {}, {}
    llm.runner.model.layer_probe = \
        lambda r, x: trail.__setitem__(r, x.detach().float().cpu().clone())
    run_steps(llm, cut("a", toks, [19]), cfg["vocab"])
    oracle.forward(cfg, w, toks, probe=lambda i, x: want.__setitem__(i, x))
    assert len(trail) == len(want) == 4
    tol = 2e-4 if dtype == "float32" else 6e-2
    for r in want:
        a, b = trail[r].double(), want[r]
        assert float((a - b).norm() / b.norm()) < tol, r


@pytest.mark.parametrize("device,dtype", DEVICES)
def test_prefill_decode_and_portions(device, dtype):
    """Whole prompt == prompt + token-by-token decoding == portions of
    many sizes (down to two tokens and one), at every position: the
    windows (9 and 17 keys) are crossed inside portions, at their starts
    and by decoded tokens; the recurrent state is handed from portion to
    portion."""
    cfg = make_config(stack_for(dtype), width=40, vocab=90, streams=3)
    w = make_weights(cfg, 3)
    llm = engine(save_model(cfg, w), device, dtype)
    toks = tokens_for(cfg, 61, 4)
    plans = {
        "whole": [61],
        "decode": [20] + [1] * 41,
        "parts": [2, 3, 2, 7, 1, 16, 5, 2, 17, 4, 2],
        "pairs": [2] * 30 + [1],
    }
    steps = []
    for rid, sizes in plans.items():
        steps += cut(rid, toks, sizes)
    got = run_steps(llm, steps, cfg["vocab"])
    check_against_oracle(cfg, w, got, {r: toks for r in plans}, TOL[dtype])


@pytest.mark.parametrize("device,dtype", DEVICES)
def test_mixed_batches_recycle_pages_and_slots(device, dtype):
    """Unequal requests batched together (portions beside single decode
    tokens) equal each request alone; the pool holds 10 pages and 3
    state slots, so later requests land on freed pages and on slots
    that still hold another sequence's state."""
    cfg = make_config(stack_for(dtype), width=32, vocab=64, streams=2)
    w = make_weights(cfg, 5)
    llm = engine(save_model(cfg, w), device, dtype, max_tokens=160, slots=3)
    P = {c: tokens_for(cfg, n, 10 + i)
         for i, (c, n) in enumerate([("a", 50), ("b", 9), ("c", 33),
                                     ("d", 21), ("e", 47), ("f", 3)])}
    steps = [
        {"entries": [("a", P["a"][:18], [0, 17]), ("b", P["b"][:2], [1])]},
        {"entries": [("b", P["b"][2:3], [0]), ("a", P["a"][18:33], [14]),
                     ("c", P["c"][:30], [0, 15, 16, 29])]},
        {"entries": [("c", P["c"][30:31], [0]), ("b", P["b"][3:9], [5]),
                     ("a", P["a"][33:34], [0])], "end": ["b"]},
        {"entries": [("a", P["a"][34:35], [0]), ("c", P["c"][31:33], [0, 1]),
                     ("d", P["d"][:21], [0, 15, 20])], "end": ["c", "d"]},
        # e and f take over the pages and slots of b, c, d
        {"entries": [("e", P["e"][:31], [15, 16, 30]), ("a", P["a"][35:36],
                                                        [0]),
                     ("f", P["f"][:3], [0, 1, 2])], "end": ["f"]},
        {"entries": [("a", P["a"][36:50], [13]), ("e", P["e"][31:32], [0])],
         "end": ["a"]},
        {"entries": [("e", P["e"][32:47], list(range(15)))], "end": ["e"]},
        # a again on recycled pages and a used slot: same answers
        {"entries": [("a#2", P["a"][:50], [0, 17, 32, 49])], "end": ["a#2"]},
    ]
    used, slots_seen = set(), []
    mm = llm.scheduler.mm
    orig = mm._allocate_fresh

    def spy(n):
        pages = orig(n)
        spy.reused |= used & set(pages)
        used.update(pages)
        return pages
    spy.reused = set()
    mm._allocate_fresh = spy
    pool = llm.runner.ssm_pool
    ensure = pool.ensure

    def spy_slot(seq):
        s = ensure(seq)
        slots_seen.append((seq.seq_id, s))
        return s
    pool.ensure = spy_slot
    got = run_steps(llm, steps, cfg["vocab"])
    assert spy.reused, "the schedule was meant to recycle pages"
    owners = {}
    for sid, s in slots_seen:
        owners.setdefault(s, set()).add(sid)
    assert any(len(v) > 1 for v in owners.values()), \
        "the schedule was meant to recycle state slots"
    check_against_oracle(cfg, w, got, P, TOL[dtype])


@pytest.mark.parametrize("device,dtype", DEVICES)
def test_long_decoding(device, dtype):
    """A short prompt, then 150 tokens decoded one by one: ten pages of
    context grow under the decode path, the windows slide over decoded
    tokens only, the state is carried 150 times; every position."""
    cfg = make_config(stack_for(dtype, [
        parallel(heads=4, kv_heads=2, dim=8, vdim=8, window=33,
                 mlp=moe_ff()),
        latent(mlp=moe_ff(experts=3, top=2, shared=0)),
        parallel(heads=2, kv_heads=1, dim=16, vdim=4, rot_dims=6,
                 window=16, gru=9)]), width=24, vocab=40, streams=2)
    w = make_weights(cfg, 9)
    llm = engine(save_model(cfg, w), device, dtype)
    toks = tokens_for(cfg, 156, 11)
    got = run_steps(llm, cut("a", toks, [6] + [1] * 150), cfg["vocab"])
    check_against_oracle(cfg, w, got, {"a": toks}, TOL[dtype])


def _paged(k, v, perm, page, npages):
    L, G, D = k.shape
    kc = torch.zeros(npages, page, G, D)
    vc = torch.zeros(npages, page, G, v.shape[2])
    pos = torch.arange(L)
    kc[perm[pos // page], pos % page] = k
    vc[perm[pos // page], pos % page] = v
    return kc, vc


@pytest.mark.parametrize("dims", [(8, 12, 4, 2), (64, 64, 8, 1),
                                  (128, 128, 4, 2), (24, 8, 3, 3)],
                         ids=["d8", "d64-gqa8", "d128", "d24-mha"])
@pytest.mark.parametrize("device,dtype", DEVICES)
def test_planted_key_at_the_window_edges(device, dtype, dims):
    """ops.window_attention with one key whose score towers over all
    others (through the tanh cap) and a value of 100: the query returns
    it exactly when the key lies inside the window — just inside and
    just outside the edge, at page borders, at the query's own place,
    far back under a wide window — for a query that ends a portion and
    for a decoded token; a large learned sink score on one head
    swallows that head's output."""
    from gllm_amd import ops
    tdt = getattr(torch, dtype)
    page = 16
    D, Dv, H, G = dims
    L = 300
    g = torch.Generator().manual_seed(7)
    npages = 64
    perm = torch.randperm(npages, generator=g)[:-(-L // page)]
    bt = perm.to(torch.int32)[None].to(device)
    sinks = torch.zeros(H)
    sinks[0] = 60.0          # head 0: the sink outweighs every key
    cap = 40.0

    def run(i, j, q_len, window):
        k = 0.05 * torch.randn(L, G, D, generator=g)
        v = torch.randn(L, G, Dv, generator=g)
        q = 0.05 * torch.randn(q_len, H, D, generator=g)
        k[j, :, 0] = 30.0
        q[-1, :, 0] = 30.0
        v[j] = 100.0
        kc, vc = _paged(k, v, perm, page, npages)
        out = ops.window_attention(
            q.reshape(q_len, H * D).to(tdt).to(device), None,
            kc.to(tdt).to(device), vc.to(tdt).to(device), bt,
            torch.tensor([i + 1], dtype=torch.int32, device=device),
            torch.tensor([0, q_len], dtype=torch.int32, device=device),
            1.0, window, 0, False, q_len, sinks=sinks.to(device),
            softcap=cap)
        return out[-1].float().cpu().view(H, Dv)

    for q_len in (1, 23, 40):
        for i in (299, 271, 255, 256):
            for window, j, seen in [
                    (0, 0, True), (0, i - 200, True), (48, i, True),
                    (48, i - 47, True), (48, i - 48, False),
                    (48, i - 49, False), (17, i - 16, True),
                    (17, i - 17, False), (1, i, True), (1, i - 1, False),
                    (250, i - 249, True), (250, i - 250, False),
                    (48, i + 1, False)]:
                if j >= L:
                    continue
                o = run(i, j, q_len, window)
                assert o[0].abs().max() < 1.0, (q_len, i, window, j)
                for h in range(1, H):
                    if seen:
                        assert (o[h] - 100.0).abs().max() < 1.0, \
                            (q_len, i, window, j, h, o[h])
                    else:
                        assert o[h].abs().max() < 10.0, \
                            (q_len, i, window, j, h)


@pytest.mark.parametrize("device,dtype", DEVICES)
def test_sink_and_cap_take_their_share(device, dtype):
    """Zero queries give every visible key weight 1 and the sink weight
    exp(sink_h): out = sum(v) / (n + exp(sink_h)); a huge score is held
    at the cap: with one key, out = v / (1 + exp(sink - cap))."""
    from gllm_amd import ops
    tdt = getattr(torch, dtype)
    page, G, H, D, L = 16, 1, 2, 4, 21
    g = torch.Generator().manual_seed(8)
    kc = torch.randn(4, page, G, D, generator=g)
    vc = torch.randn(4, page, G, D, generator=g).to(tdt).float()
    bt = torch.tensor([[2, 0, 3, 1]], dtype=torch.int32, device=device)
    sink = torch.tensor([0.7, -1.3])
    args = (kc.to(tdt).to(device), vc.to(tdt).to(device), bt,
            torch.tensor([L], dtype=torch.int32, device=device),
            torch.tensor([0, L], dtype=torch.int32, device=device))
    vs = torch.cat([vc[2], vc[0]])[:L, 0]
    tol = 1e-5 if dtype == "float32" else 2e-2
    out = ops.window_attention(
        torch.zeros(L, H * D).to(tdt).to(device), None, *args, 0.5, 6, 0,
        False, L, sinks=sink.to(device), softcap=3.0
    ).float().cpu().view(L, H, D)
    for i in (0, 1, 5, 6, 15, 16, 20):
        lo = max(0, i - 5)
        for h in range(H):
            want = vs[lo:i + 1].sum(0) / (i + 1 - lo
                                          + math.exp(float(sink[h])))
            assert (out[i, h] - want).abs().max() < tol, (i, h)
    # window 1: the key of position i is k_i itself; q = 50 * k_i
    kq = torch.cat([kc[2], kc[0]])[:L, 0].to(tdt).float()
    q = (50.0 * kq)[:, None, :].repeat(1, H, 1).reshape(L, H * D)
    out = ops.window_attention(
        q.to(tdt).to(device), None, *args, 1.0, 1, 0, False, L,
        sinks=sink.to(device), softcap=2.0).float().cpu().view(L, H, D)
    for i in (0, 7, 20):
        raw = float((q[i, :D].to(tdt).float() * kq[i]).sum())
        s = 2.0 * math.tanh(raw / 2.0)
        for h in range(H):
            want = vs[i] / (1.0 + math.exp(float(sink[h]) - s))
            assert (out[i, h] - want).abs().max() < 5 * tol, (i, h)


@pytest.mark.parametrize("device,dtype", DEVICES)
def test_rotated_values_depend_on_distance_only(device, dtype):
    """A value stored turned by its position j and read turned back by
    the query's position i arrives turned by j - i: with one visible key
    per query (window 1 sees itself) the value comes back unchanged,
    and for a planted key at distance d the head returns the value
    turned by -d, wherever the pair sits in the sequence."""
    from gllm_amd import ops
    from gllm_amd.layers.rotary import PairRotary
    tdt = getattr(torch, dtype)
    H = G = 1
    D, Dv, page, L = 4, 6, 16, 90
    rot = PairRotary(Dv, 50.0)
    freqs = rot.freqs.to(device)
    g = torch.Generator().manual_seed(3)
    v = torch.randn(L, Dv, generator=g).to(tdt)
    k = torch.zeros(L, D)
    q = torch.zeros(L, D)
    for far, d in ((False, 0), (True, 37)):
        kc = torch.zeros(8, page, G, D, dtype=tdt, device=device)
        vc = torch.zeros(8, page, G, Dv, dtype=tdt, device=device)
        pos = torch.arange(L, device=device)
        slots = pos + 2 * page
        bt = torch.tensor([[2, 3, 4, 5, 6, 7]], dtype=torch.int32,
                          device=device)
        kk, qq = k.clone(), q.clone()
        if far:
            kk[40, 0] = 30.0
            qq[40 + d, 0] = 30.0
        qd = qq.to(tdt).to(device)
        ops.qk_norm_rope_store(
            qd, kk.to(tdt).to(device), v.to(device), None, None, pos, slots,
            freqs, 1.0, 0, kc, vc, H, G, D, Dv, 1e-5, do_norm=False,
            v_freqs=freqs)
        o = ops.window_attention(
            qd, None, kc, vc, bt,
            torch.tensor([L], dtype=torch.int32, device=device),
            torch.tensor([0, L], dtype=torch.int32, device=device), 1.0,
            0 if far else 1, 0, False, L)
        o = ops.rotate_scale_rows(o, pos, freqs, H, Dv, -1.0, 2.0)
        o = o.float().cpu()
        tol = 1e-4 if dtype == "float32" else 6e-2
        if not far:
            assert (o - 2.0 * v.float()).abs().max() < tol
        else:
            ang = -d * rot.freqs.float()
            a, b = v[40].float()[0::2], v[40].float()[1::2]
            want = torch.stack([a * ang.cos() - b * ang.sin(),
                                b * ang.cos() + a * ang.sin()], -1).flatten()
            assert (o[40 + d] - 2.0 * want).abs().max() < 3 * tol


@pytest.mark.parametrize("device,dtype", DEVICES)
def test_mingru_state_carries_and_restarts(device, dtype):
    """ops.mingru_varlen: a ragged batch in one launch equals each
    sequence stepped token by token in float64; a continued sequence
    starts from its slot, a new one from zero whatever its slot holds;
    long portions (the folded segments) and single tokens alike."""
    from gllm_amd import ops
    tdt = getattr(torch, dtype)
    C = 37
    g = torch.Generator().manual_seed(5)
    lens = [1, 70, 2, 333, 17]
    T = sum(lens)
    zx = torch.randn(T, 2 * C, generator=g).to(tdt)
    gp = torch.randn(T, C, generator=g).to(tdt)
    state = torch.randn(7, C, generator=g)
    slots = torch.tensor([5, 0, 3, 6, 1])
    init = torch.tensor([1, 0, 1, 1, 0], dtype=torch.int32)
    qsl = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32)
    st = state.clone().to(device)
    buf = torch.zeros(T, C + 3, dtype=tdt, device=device)
    ops.mingru_varlen(zx.to(device), gp.to(device), st, slots.to(device),
                      init.to(device), qsl.to(device), 1.5, max(lens),
                      out=buf[:, 3:])
    out = buf[:, 3:].float().cpu()
    assert float(buf[:, :3].abs().max()) == 0.0
    want = torch.zeros(T, C, dtype=torch.float64)
    final = state.double().clone()
    z = torch.sigmoid(zx[:, :C].double())
    u = zx[:, C:].double()
    cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    gg = gp.double()
    for b, n in enumerate(lens):
        S = final[slots[b]].clone() if init[b] else torch.zeros(
            C, dtype=torch.float64)
        for t in range(int(qsl[b]), int(qsl[b + 1])):
            S = (1 - z[t]) * S + z[t] * cand[t]
            want[t] = 1.5 * S * gg[t] * torch.sigmoid(gg[t])
        final[slots[b]] = S
    tol = 1e-5 if dtype == "float32" else 3e-2
    assert (out.double() - want).abs().max() < tol
    assert (st.cpu().double() - final).abs().max() < 1e-5
    # many sequences x many channels: the wider workgroup shapes
    for B, C2 in ((40, 512), (20, 512)):
        lens2 = [9 + (7 * b) % 50 for b in range(B)]
        T2 = sum(lens2)
        zx2 = torch.randn(T2, 2 * C2, generator=g).to(tdt)
        gp2 = torch.randn(T2, C2, generator=g).to(tdt)
        st2 = torch.zeros(B + 1, C2, device=device)
        qsl2 = torch.tensor([0] + list(np.cumsum(lens2)), dtype=torch.int32)
        o2 = ops.mingru_varlen(
            zx2.to(device), gp2.to(device), st2,
            torch.arange(B).to(device),
            torch.zeros(B, dtype=torch.int32, device=device),
            qsl2.to(device), 1.0, max(lens2)).float().cpu().double()
        z2 = torch.sigmoid(zx2[:, :C2].double())
        u2 = zx2[:, C2:].double()
        c2 = torch.where(u2 >= 0, u2 + 0.5, torch.sigmoid(u2))
        g2 = gp2.double()
        for b in (0, B // 2, B - 1):
            S = torch.zeros(C2, dtype=torch.float64)
            for t in range(int(qsl2[b]), int(qsl2[b + 1])):
                S = (1 - z2[t]) * S + z2[t] * c2[t]
                assert (o2[t] - S * g2[t] * torch.sigmoid(g2[t])
                        ).abs().max() < tol, (B, b, t)
            assert (st2[b].cpu().double() - S).abs().max() < 1e-5
    # decode-only batch over the same slots
    zx1, gp1 = zx[:5].to(device), gp[:5].to(device)
    st2 = st.clone()
    o1 = ops.mingru_varlen(zx1, gp1, st2, slots.to(device),
                           torch.ones(5, dtype=torch.int32, device=device),
                           torch.arange(6, dtype=torch.int32, device=device),
                           1.0, 1).float().cpu()
    for b in range(5):
        S = (1 - z[b]) * final[slots[b]] + z[b] * cand[b]
        assert (o1[b].double() - S * gg[b] * torch.sigmoid(gg[b])
                ).abs().max() < tol
        assert (st2[slots[b]].cpu().double() - S).abs().max() < 1e-5


@pytest.mark.parametrize("device,dtype", DEVICES)
def test_hyper_streams_op(device, dtype):
    """ops.hyper_streams against the equations in float64: write with
    and without the gated second result, fused read of the updated
    streams, read alone; streams 1, 2 and 5, a width off the vector
    size."""
    from gllm_amd import ops
    tdt = getattr(torch, dtype)
    g = torch.Generator().manual_seed(6)
    for S, T, W in ((1, 5, 24), (2, 9, 36), (5, 3, 70)):
        xs = torch.randn(S, T, W, generator=g)
        y = torch.randn(T, W + 2, generator=g).to(tdt)[:, 1:W + 1]
        y2 = torch.randn(T, W, generator=g).to(tdt)
        gate = torch.randn(T, 3, generator=g).to(tdt)[:, 1:2]
        mix = torch.randn(S, S, generator=g)
        a, b = torch.randn(S, generator=g), torch.randn(S, generator=g)
        gain = torch.tensor([1.3])
        for with2 in (False, True):
            cur = xs.clone().to(device)
            h = ops.hyper_streams(
                cur, y.to(device), y2.to(device) if with2 else None,
                gate.to(device) if with2 else None, mix.to(device),
                b.to(device), read=(a.to(device), gain.to(device), 1e-5),
                dtype=tdt)
            yy = y.double()
            if with2:
                yy = yy + torch.sigmoid(gate.double()) * y2.double()
            new = torch.einsum("st,snw->tnw", mix.double(), xs.double()) \
                + b.double()[:, None, None] * yy[None]
            u = torch.einsum("s,snw->nw", a.double(), new)
            want = 1.3 * u / torch.sqrt((u * u).mean(-1, keepdim=True)
                                        + 1e-5)
            assert (cur.cpu().double() - new).abs().max() < 1e-4
            tol = 1e-4 if dtype == "float32" else 3e-2
            assert (h.float().cpu().double() - want).abs().max() < tol
            h2 = ops.hyper_streams(cur, read=(a.to(device), gain.to(device),
                                              1e-5), dtype=tdt)
            assert (h2.float() - h.float()).abs().max() < tol


@pytest.mark.parametrize("device", [
    pytest.param("cpu", id="cpu"),
    pytest.param("cuda", id="gpu", marks=pytest.mark.gpu)])
def test_routing_op(device):
    """ops.topk_then_softmax: the k largest logits in descending order,
    softmax over them alone; expert counts below, at and above a wave's
    width, k = 1, k = experts, a row with a tie (lower index first)."""
    from gllm_amd import ops
    g = torch.Generator().manual_seed(12)
    for E, k, T in ((5, 1, 7), (5, 5, 3), (64, 4, 33), (100, 8, 9),
                    (300, 2, 130), (512, 64, 2)):
        logits = torch.randn(T, E, generator=g) * 3
        w, ids = ops.topk_then_softmax(logits.to(device), k)
        w, ids = w.cpu(), ids.cpu().long()
        vals, want = torch.topk(logits, k, dim=-1)
        assert torch.equal(ids, want), (E, k)
        assert (w - torch.softmax(vals, -1)).abs().max() < 1e-6
        assert ids.dtype == torch.int64 and w.dtype == torch.float32
    tie = torch.tensor([[0.5, 2.0, -1.0, 2.0, 2.0, 0.0]])
    w, ids = ops.topk_then_softmax(tie.to(device), 2)
    assert sorted(ids.cpu().tolist()[0]) == [1, 3] or device == "cpu"
    assert (w.cpu() - 0.5).abs().max() < 1e-6


@pytest.mark.parametrize("graph", [False, True], ids=["eager", "graph"])
@pytest.mark.parametrize("device,dtype", DEVICES)
def test_greedy_generation_through_the_scheduler(device, dtype, graph):
    """LLM.generate (scheduler policy, chunked prefill, sampler) picks
    the oracle's greedy tokens; with ``graph`` the decode steps replay
    captured hipGraph buckets (bf16 on the GPU only), interleaved with
    the eager prefill steps of the later prompts."""
    if graph and (device, dtype) != ("cuda", "bfloat16"):
        pytest.skip("decode graphs are captured for bf16 on the GPU")
    from gllm_amd.config import EngineConfig
    from gllm_amd.engine.llm import LLM
    from gllm_amd.sequence import SamplingParams
    cfg = make_config(stack_for(dtype), width=32, vocab=48, streams=2)
    w = make_weights(cfg, 14)
    d = save_model(cfg, w)
    config = EngineConfig(model=d, dtype=dtype, device=device, page_size=16,
                          maxp=16, maxd=8, use_graph=graph, max_graph_bs=8,
                          model_max_length=256, enable_overlap=False)
    llm = LLM(config=config, num_pages_override=64)
    assert (llm.runner.graph_runner is not None) == graph
    prompts = [tokens_for(cfg, n, 20 + n) for n in (5, 37, 18)]
    outs = llm.generate(prompts, SamplingParams(
        temperature=0.0, max_tokens=12, ignore_eos=True))
    margin = 0.05 if dtype == "float32" else 0.5
    checked = 0
    for p, o in zip(prompts, outs):
        seq = list(p)
        for tok in o.token_ids:
            logits = oracle.forward(cfg, w, seq)[-1]
            top2 = torch.topk(logits, 2).values
            if float(top2[0] - top2[1]) >= margin:
                # (a near-tie proves nothing either way: follow the engine)
                assert tok == int(logits.argmax()), (len(seq), tok)
                checked += 1
            seq.append(tok)
    # (bf16 needs a wide margin to call a token decided; fewer qualify)
    assert checked >= (8 if dtype == "float32" else 3)


@pytest.mark.parametrize("device,dtype", DEVICES)
def test_prefix_cache_hit_restores_state(device, dtype):
    """A second prompt that shares two full pages with an earlier one
    re-uses the cached K/V and latent pages and the minGRU state
    snapshot taken at that page boundary; its greedy continuation still
    matches the oracle."""
    from gllm_amd.config import EngineConfig
    from gllm_amd.engine.llm import LLM
    from gllm_amd.sequence import SamplingParams
    cfg = make_config(stack_for(dtype), width=32, vocab=48, streams=2)
    w = make_weights(cfg, 21)
    config = EngineConfig(model=save_model(cfg, w), dtype=dtype,
                          device=device, page_size=16, maxp=16, maxd=8,
                          use_graph=False, enable_overlap=False,
                          enable_prefix_caching=True)
    llm = LLM(config=config, num_pages_override=64)
    first = tokens_for(cfg, 48, 31)
    second = first[:32] + tokens_for(cfg, 9, 32)
    sp = SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True)
    llm.generate([first], sp)
    hit_before = llm.runner.memory_manager.hit_tokens
    out = llm.generate([second], sp)[0]
    assert llm.runner.memory_manager.hit_tokens - hit_before == 32
    margin = 0.05 if dtype == "float32" else 0.5
    seq, checked = list(second), 0
    for tok in out.token_ids:
        logits = oracle.forward(cfg, w, seq)[-1]
        top2 = torch.topk(logits, 2).values
        if float(top2[0] - top2[1]) >= margin:
            assert tok == int(logits.argmax()), (len(seq), tok)
            checked += 1
        seq.append(tok)
    # (bf16 needs a wide margin to call a token decided; few qualify)
    assert checked >= (3 if dtype == "float32" else 1)


def test_config_and_registry():
    """The loader picks the class from config.json's architecture key;
    a parallel layer owns a K/V cache and a state entry, a latent layer
    one cached row per token, a kv_from layer nothing."""
    from gllm_amd.config import EngineConfig
    from gllm_amd.models.loader import load_model
    cfg = make_config(STACK, width=32, vocab=48, streams=3)
    d = save_model(cfg, make_weights(cfg, 15))
    model, _ = load_model(EngineConfig(model=d, dtype="float32",
                                       device="cpu"))
    assert type(model).__name__ == "GopetarForCausalLM"
    assert model.kv_layer_shapes == [(1, 12, 0), (2, 16, 12), (3, 10, 16)]
    assert [lay.mix.attn.layer_idx for lay in model.layers] == [0, 1, 0, 2]
    assert [s.state_shape for s in model.ssm_spec.layers] == [(20,), (13,)]
    bad = make_config([latent(kv_from=0)])
    with pytest.raises(ValueError):
        load_model(EngineConfig(model=save_model(bad, {}), dtype="float32",
                                device="cpu", load_format="dummy"))
    with pytest.raises(KeyError):
        w = make_weights(cfg, 15)
        w["l0.mix.left.q"] = torch.zeros(2, 2, dtype=torch.bfloat16)
        load_model(EngineConfig(model=save_model(cfg, w), dtype="float32",
                                device="cpu"))


def test_scaled_frequencies():
    """PairRotary's wavelength rule against the oracle's, for pairs on
    both sides of the blend and inside it."""
    from gllm_amd.layers.rotary import PairRotary
    for dims, base in ((8, 100.0), (16, 5000.0)):
        got = PairRotary(dims, base, SCALING).freqs
        plain = oracle.pair_freqs(dims, base)
        want = oracle.scaled_freqs(plain, SCALING)
        assert torch.allclose(got, want, rtol=1e-12, atol=0)
        moved = (want != plain)
        assert moved.any() and not moved.all()
