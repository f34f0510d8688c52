"""Sofunex decoder: the engine (scheduler, paged KV pool, state pool,
batch builder, ops) against the plain float64 oracle in
sofunex_oracle.py.

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

import sofunex_oracle as oracle

DEVICES = [pytest.param("cpu", "float32", id="cpu-f32"),
           pytest.param("cuda", "float32", id="gpu-f32",
                        marks=pytest.mark.gpu),
           pytest.param("cuda", "bfloat16", id="gpu-bf16",
                        marks=pytest.mark.gpu)]
TOL = {"float32": 3e-4, "bfloat16": 8e-2}


# ------------------------------------------------------------------ models
def dense_ff(ff=40):
    return {"kind": "dense", "ff": ff}


def moe_ff(experts=6, top=2, ff=16, groups=(3, 2), scale=1.7, shared=24):
    router = {"experts": experts, "top": top, "scale": scale}
    if groups:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    mlp = {"kind": "moe", "expert": {"ff": ff}, "router": router}
    if shared:
        mlp["shared"] = {"ff": shared}
    return mlp


def parallel(heads=4, kv_heads=2, dim=16, vdim=12, window=9, rot_dims=8,
             base=100.0, factor=3.0, scale=0.3, conv=3, rheads=3, rdim=12,
             rank=5, left_scale=0.7, right_scale=1.3, mlp=None):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
            "scale": scale}
    if conv:
        left["conv"] = conv
    if window:
        left["mask"] = {"size": window}
    if rot_dims is not None:
        left["rot"] = {"dims": rot_dims, "base": base}
        if factor:
            left["rot"]["scaling"] = {"factor": factor}
    return {"type": "parallel", "mlp": mlp, "_rank": rank,
            "mixer": {"left": left, "left_scale": left_scale,
                      "right": {"heads": rheads, "dim": rdim},
                      "right_scale": right_scale}}


def make_config(layers, width=32, vocab=70, eps=1e-5, embed_scale=3.0,
                mult=0.4, loop=None):
    cfg = {"architecture": "Sofunex", "embedding": {"scale": embed_scale},
           "layers": layers, "norm": {"eps": eps}, "residual_mult": mult,
           "vocab": vocab, "width": width}
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def make_weights(cfg, seed):
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]
    w = {}

    def lin(name, out, inp, gain=1.0):
        w[name] = torch.randn(out, inp, generator=g) * gain / inp ** 0.5

    def vec(name, n, gain=0.5, mean=0.0):
        w[name] = mean + gain * torch.randn(n, generator=g)

    w["embed"] = torch.randn(cfg["vocab"], W, generator=g) / 3.0
    vec("final.norm", W, 0.2, 1.0)
    lin("head", cfg["vocab"], W)
    if cfg.get("loop"):
        w["loop.step"] = 0.5 * torch.randn(cfg["loop"]["times"], W,
                                           generator=g)
    for i, layer in enumerate(cfg["layers"]):
        p = "l%d." % i
        m = layer["mixer"]
        for n in ("norm1", "norm1b"):
            vec(p + n, W, 0.2, 1.0)
        w[p + "shift"] = torch.rand(W, generator=g)
        a, r = m["left"], m["right"]
        H, G, D, Dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
        for n, rows in (("q", H * D), ("k", G * D), ("v", G * Dv)):
            lin(p + "mix.left." + n, rows, W, 2.0 if n != "v" else 1.0)
            vec(p + "mix.left.%s.b" % n, rows)
            if a.get("conv"):
                w[p + "mix.left.%s.conv" % n] = torch.randn(
                    rows, a["conv"], generator=g) / a["conv"] ** 0.5
        vec(p + "mix.left.q.norm", H * D, 0.3, 1.0)
        vec(p + "mix.left.k.norm", G * D, 0.3, 1.0)
        lin(p + "mix.left.o", W, H * Dv)
        vec(p + "mix.left.o.b", W)
        R = r["heads"] * r["dim"]
        for n in ("r", "k", "v", "g", "a"):
            lin(p + "mix.right." + n, R, W, 2.0)
        vec(p + "mix.right.a.b", R)
        lin(p + "mix.right.w1", layer["_rank"], W, 2.0)
        lin(p + "mix.right.w2", R, layer["_rank"], 3.0)
        vec(p + "mix.right.w0", R, 1.0)
        vec(p + "mix.right.norm", R, 0.3, 1.0)
        lin(p + "mix.right.o", W, R)
        mlp = layer.get("mlp")
        if not mlp:
            continue
        for n in ("norm2", "norm2b"):
            vec(p + n, W, 0.2, 1.0)
        if mlp["kind"] == "dense":
            lin(p + "mlp.gate", mlp["ff"], W, 2.0)
            lin(p + "mlp.up", mlp["ff"], W, 2.0)
            lin(p + "mlp.down", W, mlp["ff"])
            continue
        E, ff = mlp["router"]["experts"], mlp["expert"]["ff"]
        lin(p + "mlp.router", E, W, 3.0)
        w[p + "mlp.correction"] = 0.3 * torch.randn(E, generator=g)
        for e in range(E):
            lin(p + "mlp.e%d.gate" % e, ff, W, 2.0)
            lin(p + "mlp.e%d.up" % e, ff, W, 2.0)
            lin(p + "mlp.e%d.down" % e, W, ff)
        if mlp.get("shared"):
            fs = mlp["shared"]["ff"]
            lin(p + "mlp.shared.gate", fs, W, 2.0)
            lin(p + "mlp.shared.up", fs, W, 2.0)
            lin(p + "mlp.shared.down", W, fs)
    out = {k: v.to(torch.bfloat16).contiguous() for k, v in w.items()}
    for k in list(out):
        if k.endswith("mlp.correction"):
            # a correction that is exact in both number formats
            out[k] = out[k].float().to(torch.bfloat16)
    return out


def clean(cfg):
    """config.json as a checkpoint would carry it (the decay rank is
    the row count of w1, not a config key)."""
    c = json.loads(json.dumps(cfg))
    for lay in c["layers"]:
        lay.pop("_rank", None)
    return c


def save_model(cfg, weights):
    from safetensors.torch import save_file
    d = tempfile.mkdtemp(prefix="sofunex_test_")
    with open(os.path.join(d, "config.json"), "w") as f:
        json.dump(clean(cfg), f)
    save_file(weights, os.path.join(d, "model.safetensors"))
    return d


def f64(weights):
    return {k: v.to(torch.float64) for k, v in weights.items()}


# two different layers looped twice with a third behind them, an MoE
# with group limits, a dense layer and one without feed-forward
STACK = [parallel(mlp=dense_ff()),
         parallel(heads=3, kv_heads=3, dim=10, vdim=16, window=17,
                  rot_dims=10, factor=None, conv=2, rheads=2, rdim=20,
                  rank=3, mlp=moe_ff()),
         parallel(heads=2, kv_heads=1, dim=8, vdim=8, window=5, rot_dims=4,
                  conv=4, rheads=4, rdim=8, rank=7, left_scale=1.0,
                  right_scale=1.0)]
LOOP = (0, 2, 2)


def stack_for(dtype, layers=None):
    """fp32 runs route for real. In bf16 the 16-bit rounding of a
    router's input flips a close top-k call now and then, and a flip
    changes keys and the recurrent state that every later position
    reads. So the multi-layer bf16 runs use every expert (top =
    experts, one group: the grouped GEMM and the routing weights still
    run, nothing discrete is left); discrete routing in bf16 is covered
    by the one-layer models of test_each_mechanism_alone."""
    layers = STACK if layers is None else layers
    if dtype != "bfloat16":
        return layers
    out = []
    for lay in layers:
        if lay.get("mlp") and lay["mlp"]["kind"] == "moe":
            mlp = dict(lay["mlp"])
            router = dict(mlp["router"], top=mlp["router"]["experts"])
            router.pop("groups", None)
            mlp["router"] = router
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
    out = tempfile.mkdtemp(prefix="sofunex_out_")
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
    W = f64(weights)
    for rid, rows in got.items():
        key = tuple(prompts[rid.split("#")[0]])
        if key not in refs:
            refs[key] = oracle.forward(clean(cfg), W, list(key)).numpy()
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
    "plain": ([parallel()], None),
    "mha-fullrot-unscaled-wide-window": (
        [parallel(heads=2, kv_heads=2, dim=8, vdim=8, rot_dims=8,
                  factor=None, window=200)], None),
    "mqa-norot-window1-noconv": (
        [parallel(heads=3, kv_heads=1, dim=12, vdim=6, rot_dims=None,
                  window=1, conv=None)], None),
    "rot0-nowindow-taps5": (
        [parallel(rot_dims=0, vdim=20, window=None, conv=5)], None),
    "one-tap": ([parallel(conv=1, rdim=16)], None),
    "right-one-head-odd-dim": (
        [parallel(rheads=1, rdim=7, rank=1)], None),
    "right-dim40-scales-one": (
        [parallel(rheads=2, rdim=40, rank=9, left_scale=1.0,
                  right_scale=1.0)], None),
    "left-off": ([parallel(left_scale=0.0, right_scale=0.9)], None),
    "right-off": ([parallel(left_scale=1.2, right_scale=0.0)], None),
    "dense": ([parallel(mlp=dense_ff(36))], None),
    "moe-groups": ([parallel(mlp=moe_ff())], None),
    "moe-one-group-kept-top3": (
        [parallel(mlp=moe_ff(experts=8, top=3, groups=(2, 1), ff=8,
                             scale=1.0))], None),
    "moe-no-groups-no-shared-top1": (
        [parallel(mlp=moe_ff(experts=5, top=1, groups=None, shared=0))],
        None),
    "moe-singleton-groups": (
        [parallel(mlp=moe_ff(experts=4, top=2, groups=(4, 3), ff=24))],
        None),
    "loop-all-three-times": ([parallel(mlp=dense_ff(16))], (0, 1, 3)),
    "loop-middle-once": (
        [parallel(), parallel(rdim=8, conv=2, mlp=dense_ff(8)),
         parallel(window=4)], (1, 2, 1)),
    "loop-tail-twice": (
        [parallel(mlp=moe_ff(experts=4, top=4, groups=None)),
         parallel(window=6)], (1, 2, 2)),
    # head sizes that the bf16 MFMA prefill and split-KV decode kernels
    # serve (64 and 128), key sizes of every register tiling of the
    # recurrence (32, 64, 128)
    "d64-tiles-r32": (
        [parallel(heads=4, kv_heads=2, dim=64, vdim=64, rot_dims=16,
                  window=11, scale=0.1, rheads=2, rdim=32)], None),
    "d128-tiles-r64": (
        [parallel(heads=2, kv_heads=1, dim=128, vdim=128, rot_dims=128,
                  window=40, scale=0.07, rheads=1, rdim=64)], None),
    "r128": ([parallel(rheads=1, rdim=128, rank=4)], None),
}


@pytest.mark.parametrize("device,dtype", DEVICES)
@pytest.mark.parametrize("name", list(MECHANISMS))
@pytest.mark.parametrize("width", [32, 36], ids=["w32", "w36"])
def test_each_mechanism_alone(name, device, dtype, width):
    """Small models around one mechanism each, every position of a whole
    prompt (the first tokens included, the window passed several times).
    Width 36 is not a multiple of 8: unaligned projection rows, experts
    on the segment loop."""
    layers, loop = MECHANISMS[name]
    cfg = make_config(layers, width=width, loop=loop)
    w = make_weights(cfg, 1)
    llm = engine(save_model(cfg, w), device, dtype)
    toks = tokens_for(cfg, 37, 2)
    # the whole prompt, then the same prompt as a portion and decoding
    # (a second request: other pages, the decode kernels)
    steps = cut("a", toks, [37]) + cut("b", toks, [30] + [1] * 7)
    got = run_steps(llm, steps, cfg["vocab"])
    check_against_oracle(cfg, w, got, {"a": toks, "b": toks}, TOL[dtype])


@pytest.mark.parametrize("device,dtype", DEVICES)
def test_layer_trail_matches(device, dtype):
    """The residual stream after every layer run (looped layers count
    each time) against the oracle's, through the model's layer probe."""
    cfg = make_config(stack_for(dtype), width=40, vocab=90, loop=LOOP)
    w = make_weights(cfg, 21)
    llm = engine(save_model(cfg, w), device, dtype)
    toks = tokens_for(cfg, 19, 22)
    trail, want = {}, []
    llm.runner.model.layer_probe = \
        lambda r, x: trail.__setitem__(r, x.detach().float().cpu().clone())
    run_steps(llm, cut("a", toks, [19]), cfg["vocab"])
    oracle.forward(clean(cfg), f64(w), toks, probe=want)
    assert len(trail) == len(want) == 5
    tol = 2e-4 if dtype == "float32" else 6e-2
    for r, b in enumerate(want):
        a = trail[r].double()
        assert float((a - b).norm() / b.norm()) < tol, r


@pytest.mark.parametrize("device,dtype", DEVICES)
def test_prefill_decode_and_portions(device, dtype):
    """Whole prompt == prompt + token-by-token decoding == portions of
    many sizes (down to two tokens and one), at every position: the
    windows (9, 17 and 5 keys) are crossed inside portions, at their
    starts and by decoded tokens; the shifted row, the convolution's
    history (1 to 3 rows) and the recurrent state are handed from
    portion to portion, also by portions shorter than the history."""
    cfg = make_config(stack_for(dtype), width=40, vocab=90, loop=LOOP)
    w = make_weights(cfg, 3)
    llm = engine(save_model(cfg, w), device, dtype)
    toks = tokens_for(cfg, 61, 4)
    plans = {
        "whole": [61],
        "decode": [20] + [1] * 41,
        "parts": [2, 3, 2, 7, 1, 16, 5, 2, 17, 4, 2],
        "pairs": [2] * 30 + [1],
        "ones-first": [1, 1, 1, 2, 1, 55],
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
    that still hold another sequence's shifted row, convolution history
    and recurrent state."""
    cfg = make_config(stack_for(dtype), width=32, vocab=64, loop=LOOP)
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
        parallel(heads=2, kv_heads=1, dim=16, vdim=4, rot_dims=6,
                 window=16, rheads=2, rdim=16, mlp=dense_ff(24))]),
        width=24, vocab=40, loop=(1, 2, 2))
    w = make_weights(cfg, 9)
    llm = engine(save_model(cfg, w), device, dtype)
    toks = tokens_for(cfg, 156, 11)
    got = run_steps(llm, cut("a", toks, [6] + [1] * 150), cfg["vocab"])
    check_against_oracle(cfg, w, got, {"a": toks}, TOL[dtype])


@pytest.mark.parametrize("device,dtype", DEVICES)
def test_long_prompt_and_its_continuation(device, dtype):
    """A 540-token prompt in one step (the kernels that prompt-sized
    batches select), the same prompt as 515 tokens + a portion of 2 +
    single tokens, and as two long portions: the ends of the prompt and
    places around both cuts against the oracle."""
    cfg = make_config(stack_for(dtype, [
        parallel(heads=4, kv_heads=2, dim=16, vdim=8, window=70,
                 rot_dims=8, rheads=2, rdim=16, mlp=dense_ff(24)),
        parallel(heads=2, kv_heads=1, dim=64, vdim=64, window=300,
                 rot_dims=32, conv=4, rheads=1, rdim=32,
                 mlp=moe_ff(experts=4, top=2, groups=(2, 1)))]),
        width=32, vocab=50, loop=(0, 1, 2))
    w = make_weights(cfg, 17)
    llm = engine(save_model(cfg, w), device, dtype, max_tokens=1200)
    toks = tokens_for(cfg, 540, 18)

    def steps(rid, sizes):
        out, lo = [], 0
        for n in sizes:
            want = [k for k in range(n)
                    if lo + k in (0, 1, 69, 70, 71, 299, 300, 301, 511, 512,
                                  513, 514, 515, 516, 517, 530, 538, 539)]
            out.append({"entries": [(rid, toks[lo:lo + n], want)]})
            lo += n
        assert lo == 540
        out[-1]["end"] = [rid]
        return out

    got = run_steps(llm, steps("whole", [540])
                    + steps("tail", [515, 2] + [1] * 23)
                    + steps("halves", [513, 27]), cfg["vocab"])
    check_against_oracle(cfg, w, got, {r: toks for r in got}, TOL[dtype])


def _paged(k, v, perm, page, npages):
    L, G, D = k.shape
    kc = torch.zeros(npages, page, G, D)
    vc = torch.zeros(npages, page, G, v.shape[2])
    pos = torch.arange(L)
    kc[perm[pos // page], pos % page] = k
    vc[perm[pos // page], pos % page] = v
    return kc, vc


@pytest.mark.parametrize("dims", [(8, 12, 4, 2), (64, 64, 8, 1),
                                  (128, 128, 4, 2)],
                         ids=["d8", "d64-gqa8", "d128"])
@pytest.mark.parametrize("device,dtype", DEVICES)
def test_planted_key_at_the_window_edges(device, dtype, dims):
    """ops.window_attention as this family calls it (no sink, no cap)
    with one key whose score towers over all others and a value of 100:
    the query returns it exactly when the key lies inside the window —
    just inside and just outside the edge, at page borders, at the
    query's own place, far back under a wide window — for a query that
    ends a portion and for a decoded token."""
    from gllm_amd import ops
    tdt = getattr(torch, dtype)
    page = 16
    D, Dv, H, G = dims
    L = 300
    g = torch.Generator().manual_seed(7)
    npages = 64
    perm = torch.randperm(npages, generator=g)[:-(-L // page)]
    bt = perm.to(torch.int32)[None].to(device)

    def run(i, j, q_len, window):
        k = 0.05 * torch.randn(L, G, D, generator=g)
        v = torch.randn(L, G, Dv, generator=g)
        q = 0.05 * torch.randn(q_len, H, D, generator=g)
        k[j, :, 0] = 8.0
        q[-1, :, 0] = 8.0
        v[j] = 100.0
        kc, vc = _paged(k, v, perm, page, npages)
        out = ops.window_attention(
            q.reshape(q_len, H * D).to(tdt).to(device), None,
            kc.to(tdt).to(device), vc.to(tdt).to(device), bt,
            torch.tensor([i + 1], dtype=torch.int32, device=device),
            torch.tensor([0, q_len], dtype=torch.int32, device=device),
            1.0, window, 0, False, q_len)
        return out[-1].float().cpu().view(H, Dv)

    for q_len in (1, 23):
        for i in (299, 271, 255, 256):
            for window, j, seen in [
                    (0, 0, True), (0, i - 200, True), (48, i, True),
                    (48, i - 47, True), (48, i - 48, False),
                    (17, i - 16, True), (17, i - 17, False),
                    (1, i, True), (1, i - 1, False),
                    (250, i - 249, True), (250, i - 250, False)]:
                o = run(i, j, q_len, window)
                if seen:
                    assert (o - 100.0).abs().max() < 1.0, \
                        (q_len, i, window, j)
                else:
                    assert o.abs().max() < 10.0, (q_len, i, window, j)


def _rows(device, slots, init, qsl):
    return (torch.tensor(slots, dtype=torch.long, device=device),
            torch.tensor(init, dtype=torch.int32, device=device),
            torch.tensor(qsl, dtype=torch.int32, device=device))


@pytest.mark.parametrize("width", [24, 20], ids=["w24", "w20"])
@pytest.mark.parametrize("device,dtype", DEVICES)
def test_token_shift_op(device, dtype, width):
    """ops.token_shift over a ragged batch against the oracle on whole
    sequences: portions of 1, 2 and more rows, a slot that still holds
    another sequence's row is ignored by a sequence that starts there,
    and a decode-only batch rolls the state in the same launch."""
    from gllm_amd import ops
    tdt = getattr(torch, dtype)
    g = torch.Generator().manual_seed(3)
    mu = torch.rand(width, generator=g).to(tdt)
    seqs = [torch.randn(n, width, generator=g).to(tdt) for n in (9, 4, 6)]
    want = [oracle.token_shift(s.double(), mu.double()) for s in seqs]
    state = torch.full((5, width), 7.0, dtype=tdt, device=device)
    slot = [3, 0, 4]
    got = [torch.zeros_like(s) for s in seqs]
    # (portion sizes per step and sequence; 0 = not in the batch)
    plan = [(5, 1, 0), (1, 1, 2), (1, 1, 1), (2, 1, 3)]
    at = [0, 0, 0]
    for sizes in plan:
        rows, sl, init, qsl, where = [], [], [], [0], []
        for b, n in enumerate(sizes):
            if not n:
                continue
            rows.append(seqs[b][at[b]:at[b] + n])
            sl.append(slot[b])
            init.append(int(at[b] > 0))
            qsl.append(qsl[-1] + n)
            where.append((b, at[b], n))
            at[b] += n
        h = torch.cat(rows).to(device)
        s_t, i_t, q_t = _rows(device, sl, init, qsl)
        out = ops.token_shift(h, mu.to(device), state, s_t, i_t, q_t,
                              max(sizes)).cpu()
        for (b, lo, n), o0 in zip(where, qsl):
            got[b][lo:lo + n] = out[o0:o0 + n]
    assert at == [9, 4, 6]
    tol = 1e-6 if dtype == "float32" else 2e-2
    for a, b in zip(got, want):
        assert (a.double() - b).abs().max() < tol
    # the state holds each sequence's last incoming row
    for b in range(3):
        assert torch.equal(state[slot[b]].cpu(), seqs[b][-1])


@pytest.mark.parametrize("device,dtype", DEVICES)
def test_short_conv_without_activation(device, dtype):
    """ops.causal_conv_silu(activation=False) across portions shorter
    and longer than the history equals the oracle's convolution of the
    whole sequence; channel counts on both code paths (8-wide and
    scalar)."""
    from gllm_amd import ops
    tdt = getattr(torch, dtype)
    g = torch.Generator().manual_seed(4)
    for C, taps in ((24, 3), (20, 4), (16, 2), (8, 1)):
        w = (torch.randn(C, taps, generator=g) / taps ** 0.5).to(tdt)
        u = torch.randn(23, C, generator=g).to(tdt)
        want = oracle.short_conv(u.double(), w.double())
        state = torch.full((3, C, max(taps - 1, 1)), 5.0, dtype=tdt,
                           device=device)
        outs, lo = [], 0
        for n in (1, 2, 1, 7, 3, 9):
            s_t, i_t, q_t = _rows(device, [1], [int(lo > 0)], [0, n])
            outs.append(ops.causal_conv_silu(
                u[lo:lo + n].to(device), w.to(device), state, s_t, i_t, q_t,
                activation=False).cpu())
            lo += n
        got = torch.cat(outs).double()
        tol = 1e-5 if dtype == "float32" else 3e-2
        assert (got - want).abs().max() < tol, (C, taps)


@pytest.mark.parametrize("dims", [(2, 8), (3, 12), (1, 32), (2, 64),
                                  (1, 128), (1, 200)],
                         ids=["d8", "d12", "d32", "d64", "d128", "d200"])
@pytest.mark.parametrize("device,dtype", DEVICES)
def test_general_delta_rule_op(device, dtype, dims):
    """ops.general_delta_rule over a ragged batch (a long portion, short
    ones, single tokens, a slot that held another sequence) against the
    oracle's recurrence on the whole sequences."""
    from gllm_amd import ops
    tdt = getattr(torch, dtype)
    H, D = dims
    g = torch.Generator().manual_seed(5)
    c = math.exp(-0.5)
    w0 = torch.randn(H * D, generator=g).to(tdt)
    lens = (40, 5, 11)
    seqs = []
    for n in lens:
        r, k, v, wl, al = (torch.randn(n, H * D, generator=g).to(tdt)
                           for _ in range(5))
        seqs.append((r, k, v, wl, al))
    want = []
    for r, k, v, wl, al in seqs:
        n = r.shape[0]
        w = torch.exp(-c * torch.sigmoid(wl.double() + w0.double()))
        a = torch.sigmoid(al.double())
        want.append(oracle.delta_recurrence(
            r.double().view(n, H, D), k.double().view(n, H, D),
            v.double().view(n, H, D), w.view(n, H, D), a.view(n, H, D)))
    state = torch.full((4, H, D, D), 3.0, device=device)
    slot = [2, 0, 1]
    got = [torch.zeros(n, H, D) for n in lens]
    plan = [(30, 1, 0), (1, 1, 2), (2, 1, 1), (7, 2, 8)]
    at = [0, 0, 0]
    for sizes in plan:
        parts, sl, init, qsl, where = [], [], [], [0], []
        for b, n in enumerate(sizes):
            if not n:
                continue
            parts.append([x[at[b]:at[b] + n] for x in seqs[b]])
            sl.append(slot[b])
            init.append(int(at[b] > 0))
            qsl.append(qsl[-1] + n)
            where.append((b, at[b], n))
            at[b] += n
        ops5 = [torch.cat([p[i] for p in parts]).to(device)
                for i in range(5)]
        s_t, i_t, q_t = _rows(device, sl, init, qsl)
        o = ops.general_delta_rule(*ops5, w0.to(device), c, state, s_t, i_t,
                                   q_t, max(sizes)).cpu()
        for (b, lo, n), o0 in zip(where, qsl):
            got[b][lo:lo + n] = o[o0:o0 + n]
    assert at == list(lens)
    tol = 2e-4 if dtype == "float32" else 5e-2
    for a, b in zip(got, want):
        assert float((a.double() - b).norm() / b.norm()) < tol


@pytest.mark.parametrize("device,dtype", DEVICES)
def test_state_keeps_a_far_pair(device, dtype):
    """A key/value pair written at position 0 with decay 1 and removal
    rate 0 everywhere is read back unchanged 400 tokens later, through
    a prompt portion and 40 single steps (nothing in between writes:
    their values are zero); with full removal along the same key
    (a = 1) at position 200 it is gone."""
    from gllm_amd import ops
    tdt = getattr(torch, dtype)
    H, D, L = 2, 16, 400
    g = torch.Generator().manual_seed(6)

    def run(erase_at):
        k = torch.randn(L, H * D, generator=g)
        k[0] = torch.randn(H * D, generator=g)
        v = torch.zeros(L, H * D)
        v[0] = 3.0
        r = torch.zeros(L, H * D)
        # read along the first key, normalised: o = v (k0 . k0 / |k0|^2)
        k0 = k[0].view(H, D)
        r[-1] = (k0 / (k0 * k0).sum(-1, keepdim=True)).reshape(-1)
        wl = torch.full((L, H * D), -60.0)     # sigmoid -> 0, decay -> 1
        al = torch.full((L, H * D), -60.0)     # removal rate -> 0
        if erase_at is not None:
            k[erase_at] = k[0]
            al[erase_at] = 60.0
        state = torch.zeros(2, H, D, D, device=device)
        w0 = torch.zeros(H * D, dtype=tdt, device=device)
        outs, lo = [], 0
        for n in [L - 40] + [1] * 40:
            s_t, i_t, q_t = _rows(device, [1], [int(lo > 0)], [0, n])
            args = [x[lo:lo + n].to(tdt).to(device)
                    for x in (r, k, v, wl, al)]
            outs.append(ops.general_delta_rule(
                *args, w0, math.exp(-0.5), state, s_t, i_t, q_t, n).cpu())
            lo += n
        return torch.cat(outs)[-1]

    kept = run(None)
    assert (kept - 3.0).abs().max() < (1e-3 if dtype == "float32" else 0.1)
    gone = run(200)
    assert gone.abs().max() < (1e-3 if dtype == "float32" else 0.1)


@pytest.mark.parametrize("device,dtype", DEVICES)
def test_stream_rmsnorm_op(device, dtype):
    """ops.stream_rmsnorm: every combination of its parts against the
    plain formula, aligned and unaligned widths, strided sublayer rows."""
    from gllm_amd import ops
    tdt = getattr(torch, dtype)
    g = torch.Generator().manual_seed(8)
    eps = 1e-5
    for width in (32, 36, 600):
        T = 5
        x0 = torch.randn(T, width, generator=g) * 3
        wide = torch.randn(T, 2 * width + 8, generator=g).to(tdt)
        y, y2 = wide[:, :width], wide[:, width + 8:]
        wp = (1 + 0.2 * torch.randn(width, generator=g)).to(tdt)
        wn = (1 + 0.2 * torch.randn(width, generator=g)).to(tdt)
        add = torch.randn(width, generator=g)
        for use_y, use_y2, use_add, use_pre in [
                (True, False, False, True), (True, True, True, True),
                (True, True, False, False), (False, False, True, True),
                (False, False, False, True), (True, False, True, False)]:
            x = x0.clone().to(device)
            wide_d = wide.to(device)
            h = ops.stream_rmsnorm(
                x, wide_d[:, :width] if use_y else None,
                wp.to(device) if use_y else None, eps, 0.3, 0.8,
                wide_d[:, width + 8:] if use_y2 else None,
                add.to(device) if use_add else None,
                wn.to(device) if use_pre else None)
            ref = x0.double()
            if use_y:
                z = y.double() + (y2.double() if use_y2 else 0)
                ref = ref + 0.3 * oracle.unit_rms(0.8 * z, eps) * wp.double()
            if use_add:
                ref = ref + add.double()
            assert (x.cpu().double() - ref).abs().max() < 1e-4
            if use_pre:
                want = oracle.unit_rms(ref, eps) * wn.double()
                tol = 1e-4 if dtype == "float32" else 5e-2
                assert (h.cpu().double() - want).abs().max() < tol
            else:
                assert h is None


@pytest.mark.parametrize("device", [pytest.param("cpu", id="cpu"),
                                    pytest.param("cuda", id="gpu",
                                                 marks=pytest.mark.gpu)])
def test_routing_op(device):
    """ops.sigmoid_group_topk against the oracle's router: expert counts
    below, at and above a wave's width, one group, singleton groups,
    corrections that make every choice score negative (a masked expert
    must lose to a negative one: it counts as -inf, not 0), weights
    without the correction, top = all."""
    from gllm_amd import ops
    g = torch.Generator().manual_seed(12)
    for E, k, ng, keep, T, shift in (
            (6, 2, 3, 2, 7, 0.0), (10, 4, 2, 1, 33, 0.0),
            (8, 3, 2, 1, 40, -5.0), (64, 6, 8, 3, 9, -2.0),
            (5, 1, 1, 1, 3, 0.0), (4, 2, 4, 3, 11, -3.0),
            (300, 8, 10, 4, 130, 0.0), (512, 64, 4, 1, 2, 0.0),
            (12, 12, 3, 3, 5, 0.0)):
        logits = torch.randn(T, E, generator=g) * 2
        corr = torch.randn(E, generator=g) * 0.5 + shift
        w, ids = ops.sigmoid_group_topk(logits.to(device), corr.to(device),
                                        k, ng, keep, 1.9)
        w, ids = w.cpu().double(), ids.cpu().long()
        mlp = {"router": {"experts": E, "top": k, "scale": 1.9,
                          "groups": {"count": ng, "keep": keep}}}
        # the oracle's router on logits: identity "hidden" rows
        W = {"r.router": torch.eye(E, dtype=torch.float64),
             "r.correction": corr.double()}
        want_ids, want_w = oracle.route(logits.double(), mlp, W, "r.")
        assert torch.equal(ids.sort(-1)[0], want_ids.sort(-1)[0]), (E, k)
        order = ids.argsort(-1)
        worder = want_ids.argsort(-1)
        assert (w.gather(1, order) - want_w.gather(1, worder)
                ).abs().max() < 1e-5, (E, k)
    # no correction tensor, no groups
    logits = torch.randn(9, 10, generator=g)
    w, ids = ops.sigmoid_group_topk(logits.to(device), None, 3)
    s = torch.sigmoid(logits)
    assert torch.equal(ids.cpu().long().sort(-1)[0],
                       s.topk(3, -1)[1].sort(-1)[0])
    assert (w.cpu().sum(-1) - 1.0).abs().max() < 1e-5


@pytest.mark.parametrize("T", [11, 600], ids=["t11", "t600"])
@pytest.mark.parametrize("device,dtype", DEVICES)
def test_span_norm_and_unit_values(device, dtype, T):
    """ops.qk_norm_rope_store with one RMS over the whole q (k) row,
    rotate-half on a prefix of the head and unit-RMS values, against
    the oracle's pieces, rows scattered over pages in a shuffled order.
    One head is scaled up a thousandfold: a per-head norm would hide
    that, the row norm shrinks every other head. 600 rows reach the
    workgroup-per-token kernel of prompt-sized batches."""
    from gllm_amd import ops
    tdt = getattr(torch, dtype)
    g = torch.Generator().manual_seed(13)
    H, G, D, Dv, dims, eps = 4, 2, 12, 10, 8, 1e-5
    q = torch.randn(T, H * D, generator=g)
    q[:, :D] *= 1000.0
    k = torch.randn(T, G * D, generator=g)
    v = torch.randn(T, G * Dv, generator=g) * 4
    qw = 1 + 0.3 * torch.randn(H * D, generator=g)
    kw = 1 + 0.3 * torch.randn(G * D, generator=g)
    q, k, v, qw, kw = (x.to(tdt) for x in (q, k, v, qw, kw))
    pos = torch.arange(5, 5 + T)
    npages = T // 16 + 4
    slot = torch.randperm(npages * 16, generator=g)[:T]
    freqs = (50.0 ** (-2.0 * torch.arange(dims // 2, dtype=torch.float64)
                      / dims)) / 2.0
    kc = torch.zeros(npages, 16, G, D, dtype=tdt, device=device)
    vc = torch.zeros(npages, 16, G, Dv, dtype=tdt, device=device)
    q_out = torch.zeros(T, H * D, dtype=tdt, device=device)
    ops.qk_norm_rope_store(
        q.to(device), k.to(device), v.to(device), qw.to(device),
        kw.to(device), pos.to(device), slot.to(device), freqs.to(device),
        1.0, dims, kc, vc, H, G, D, Dv, eps, half_layout=True,
        norm_span=True, v_unit=True, q_out=q_out)

    def turned(x, w, heads):
        xn = oracle.unit_rms(x.double(), eps) * w.double()
        full = torch.zeros(int(pos[-1]) + 1, heads, D, dtype=torch.float64)
        full[pos] = xn.view(T, heads, D)
        return oracle.rotate_half(full, dims, 50.0, 2.0)[pos]

    tol = 1e-5 if dtype == "float32" else 3e-2
    want_q = turned(q, qw, H).reshape(T, H * D)
    assert (q_out.cpu().double() - want_q).abs().max() < tol * 40
    assert want_q[:, D:].abs().max() < 0.05   # the big head took the norm
    got_k = kc.view(-1, G, D)[slot.to(device)].cpu().double()
    assert (got_k - turned(k, kw, G)).abs().max() < tol
    got_v = vc.view(-1, G, Dv)[slot.to(device)].cpu().double()
    want_v = oracle.unit_rms(v.double().view(T, G, Dv), eps)
    assert (got_v - want_v).abs().max() < tol


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
    cfg = make_config(stack_for(dtype), width=32, vocab=48, loop=LOOP)
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
    W = f64(w)
    for p, o in zip(prompts, outs):
        seq = list(p)
        for tok in o.token_ids:
            logits = oracle.forward(clean(cfg), W, seq)[-1]
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
    re-uses the cached K/V pages and the snapshot of shifted row,
    convolution history and recurrent state taken at that page
    boundary; its greedy continuation still matches the oracle."""
    from gllm_amd.config import EngineConfig
    from gllm_amd.engine.llm import LLM
    from gllm_amd.sequence import SamplingParams
    cfg = make_config(stack_for(dtype), width=32, vocab=48, loop=LOOP)
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
    W = f64(w)
    for tok in out.token_ids:
        logits = oracle.forward(clean(cfg), W, seq)[-1]
        top2 = torch.topk(logits, 2).values
        if float(top2[0] - top2[1]) >= margin:
            assert tok == int(logits.argmax()), (len(seq), tok)
            checked += 1
        seq.append(tok)
    # (bf16 needs a wide margin to call a token decided; few qualify)
    assert checked >= (3 if dtype == "float32" else 1)


def test_config_and_registry():
    """The loader picks the class from config.json's architecture key;
    every layer RUN owns a K/V cache and a state entry (shifted row,
    convolution history, recurrent state); the decay rank comes from
    w1's rows whatever the order of the tensors; unknown tensors and a
    missing w1 raise."""
    from gllm_amd.config import EngineConfig
    from gllm_amd.models.loader import load_model
    cfg = make_config(STACK, width=32, vocab=48, loop=LOOP)
    wts = make_weights(cfg, 15)
    model, _ = load_model(EngineConfig(model=save_model(cfg, wts),
                                       dtype="float32", device="cpu"))
    assert type(model).__name__ == "SofunexForCausalLM"
    assert model.runs == [(0, 0), (1, None), (0, 1), (1, None), (2, None)]
    assert model.kv_layer_shapes == [(2, 16, 12), (3, 10, 16)] * 2 \
        + [(1, 8, 8)]
    specs = model.ssm_spec.layers
    assert [(s.conv_dim, s.conv_kernel, s.shift_dim) for s in specs] == \
        [(120, 3, 32), (108, 2, 32)] * 2 + [(32, 4, 32)]
    assert [lay.mix.rank for lay in model.layers] == [5, 3, 7]
    with pytest.raises(KeyError):
        bad = dict(wts)
        bad["l0.mix.left.sink"] = torch.zeros(4, dtype=torch.bfloat16)
        load_model(EngineConfig(model=save_model(cfg, bad), dtype="float32",
                                device="cpu"))
    with pytest.raises(KeyError):
        bad = {k: v for k, v in wts.items() if k != "l1.mix.right.w1"}
        load_model(EngineConfig(model=save_model(cfg, bad), dtype="float32",
                                device="cpu"))
    with pytest.raises(ValueError):
        load_model(EngineConfig(
            model=save_model(make_config(STACK, loop=(2, 1, 2)), {}),
            dtype="float32", device="cpu"))


def test_linear_scaling_of_frequencies():
    """HalfRotary divides every frequency by the scaling factor."""
    from gllm_amd.layers.rotary import HalfRotary
    plain = HalfRotary(8, 100.0).freqs
    assert torch.allclose(HalfRotary(8, 100.0, {"factor": 4.0}).freqs,
                          plain / 4.0, rtol=1e-15, atol=0)
    with pytest.raises(ValueError):
        HalfRotary(8, 100.0, {"factor": 2.0, "original": 64})
