"""Gukirax decoder: the engine (scheduler, paged KV pool, batch builder,
ops) against the plain float64 oracle in gukirax_oracle.py.

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

import gukirax_oracle as oracle

DEVICES = [pytest.param("cpu", "float32", id="cpu-f32"),
           pytest.param("cuda", "float32", id="gpu-f32",
                        marks=pytest.mark.gpu),
           pytest.param("cuda", "bfloat16", id="gpu-bf16",
                        marks=pytest.mark.gpu)]
TOL = {"float32": 3e-4, "bfloat16": 8e-2}


# ------------------------------------------------------------------ models
def attn(heads=4, kv_heads=2, dim=16, rot_dims=8, base=10000.0, scale=0.3):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim,
         "scale": scale}
    if rot_dims is not None:
        m["rot"] = {"dims": rot_dims, "base": base}
    return {"type": "attention", "mixer": m, "mlp": None}


def dense(layer, ff=48):
    return dict(layer, mlp={"kind": "dense", "ff": ff})


def moe(layer, experts=6, top=2, ff=16, shared=24):
    mlp = {"kind": "moe", "expert": {"ff": ff},
           "router": {"experts": experts, "top": top}}
    if shared:
        mlp["shared"] = {"ff": shared}
    return dict(layer, mlp=mlp)


def make_config(layers, width=32, vocab=70, eps=1e-5, loop=(0, 1, 1),
                logit_scale=0.7, softcap=12.0):
    cfg = {"architecture": "Gukirax", "layers": layers,
           "logit_scale": logit_scale, "logit_softcap": softcap,
           "norm": {"eps": eps}, "vocab": vocab, "width": width}
    if loop is not None:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def make_weights(cfg, seed):
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]
    w = {}

    def lin(name, out, inp, gain=1.0):
        w[name] = torch.randn(out, inp, generator=g) * gain / inp ** 0.5

    def norm(name):
        w[name] = 1.0 + 0.2 * torch.randn(W, generator=g)

    w["embed"] = torch.randn(cfg["vocab"], W, generator=g)
    norm("embed.norm")
    norm("final.norm")
    if cfg.get("loop"):
        lin("loop.in", W, 2 * W, 1.5)
    for i, layer in enumerate(cfg["layers"]):
        p = "l%d." % i
        m = layer["mixer"]
        H, G, D = m["heads"], m["kv_heads"], m["dim"]
        norm(p + "norm1")
        norm(p + "norm1b")
        lin(p + "mix.q", H * D, W, 2.0)
        lin(p + "mix.k", G * D, W, 2.0)
        lin(p + "mix.o", W, H * D)
        w[p + "mix.talk"] = torch.eye(H) + 0.4 * torch.randn(H, H,
                                                             generator=g)
        w[p + "mix.sink"] = torch.randn(H, generator=g)
        lin(p + "rg1", W, W)
        w[p + "rg1.b"] = 0.5 * torch.randn(W, generator=g)
        mlp = layer.get("mlp")
        if not mlp:
            continue
        norm(p + "norm2")
        norm(p + "norm2b")
        lin(p + "rg2", W, W)
        w[p + "rg2.b"] = 0.5 * torch.randn(W, generator=g)
        if mlp["kind"] == "dense":
            lin(p + "mlp.up", mlp["ff"], W, 1.5)
            lin(p + "mlp.down", W, mlp["ff"])
            w[p + "mlp.act"] = torch.randn(2, generator=g)
        else:
            E, ff = mlp["router"]["experts"], mlp["expert"]["ff"]
            lin(p + "mlp.router", E, W, 2.0)
            for e in range(E):
                lin(p + "mlp.e%d.up" % e, ff, W, 1.5)
                lin(p + "mlp.e%d.down" % e, W, ff)
            if mlp.get("shared"):
                lin(p + "mlp.shared.up", mlp["shared"]["ff"], W, 1.5)
                lin(p + "mlp.shared.down", W, mlp["shared"]["ff"])
    return {k: v.to(torch.bfloat16).contiguous() for k, v in w.items()}


def save_model(cfg, weights):
    from safetensors.torch import save_file
    d = tempfile.mkdtemp(prefix="gukirax_test_")
    with open(os.path.join(d, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file(weights, os.path.join(d, "model.safetensors"))
    return d


# layer 0 ahead of the loop, layers 1-2 looped three times, layer 3 after
STACK = [dense(attn(heads=2, kv_heads=2, dim=12, rot_dims=12)),
         moe(attn()),
         attn(heads=4, kv_heads=1, dim=8, rot_dims=4),
         moe(attn(heads=3, kv_heads=3, dim=20, rot_dims=None), experts=4,
             top=1, ff=8, shared=0)]
STACK_LOOP = (1, 3, 3)


# ------------------------------------------------------------------ harness
def engine(model_dir, device, dtype, max_tokens=256, slots=4, page=16):
    from gllm_amd.entrypoints.trace_replay import build_engine
    return build_engine(model_dir, dtype, max_tokens, slots, device, page)


def run_steps(llm, steps, vocab):
    """steps: [{"entries": [(rid, tokens, want)], "end": [rid]}] ->
    {rid: {position: logits}} through trace_replay.replay."""
    from gllm_amd.entrypoints.trace_replay import replay
    out = tempfile.mkdtemp(prefix="gukirax_out_")
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
@pytest.mark.parametrize("device,dtype", DEVICES)
@pytest.mark.parametrize("layers,loop", [
    ([attn()], None),
    ([attn(heads=2, kv_heads=2, dim=10, rot_dims=10)], (0, 1, 1)),
    ([attn(heads=3, kv_heads=1, dim=12, rot_dims=None)], (0, 1, 2)),
    ([dense(attn())], (0, 1, 1)),
    ([moe(attn())], (0, 1, 1)),
    ([moe(attn(), experts=3, top=3, ff=24, shared=0)], None),
    ([moe(attn(), experts=5, top=1, ff=8, shared=8)], (0, 0, 4)),
], ids=["attn-noloop", "attn-mha-fullrot", "attn-mqa-norot-twice", "dense",
        "moe", "moe-all-experts", "moe-top1-emptyloop"])
@pytest.mark.parametrize("width", [32, 36], ids=["w32", "w36"])
def test_each_mechanism_alone(layers, loop, device, dtype, width):
    """One-layer models: the mixer and each feed-forward on its own,
    every position of a whole prompt (the first tokens included). Width
    36 is not a multiple of 8: scalar norm kernels, unaligned projection
    rows, experts on the segment loop."""
    cfg = make_config(layers, width=width, loop=loop)
    w = make_weights(cfg, 1)
    llm = engine(save_model(cfg, w), device, dtype)
    toks = tokens_for(cfg, 37, 2)
    got = run_steps(llm, cut("a", toks, [37]), cfg["vocab"])
    check_against_oracle(cfg, w, got, {"a": toks}, TOL[dtype])


@pytest.mark.parametrize("device,dtype", DEVICES)
def test_layer_trail_matches(device, dtype):
    """The residual stream after every layer RUN (looped layers count
    each time) against the oracle's, through the model's layer probe."""
    cfg = make_config(STACK, width=40, vocab=90, loop=STACK_LOOP)
    w = make_weights(cfg, 21)
    llm = engine(save_model(cfg, w), device, dtype)
    toks = tokens_for(cfg, 19, 22)
    trail = {}
    llm.runner.model.layer_probe = \
        lambda r, x: trail.__setitem__(r, x.detach().float().cpu().clone())
    run_steps(llm, cut("a", toks, [19]), cfg["vocab"])
    _, want = oracle.forward(cfg, w, toks, with_layers=True)
    assert len(trail) == want.shape[0] == 1 + 2 * 3 + 1
    tol = 2e-4 if dtype == "float32" else 6e-2
    for r in range(want.shape[0]):
        a, b = trail[r].double(), want[r]
        assert float((a - b).norm() / b.norm()) < tol, r


@pytest.mark.parametrize("device,dtype", DEVICES)
def test_prefill_decode_and_portions(device, dtype):
    """Whole prompt == prompt + token-by-token decoding == portions of
    many sizes (down to two tokens and one), at every position."""
    cfg = make_config(STACK, width=40, vocab=90, loop=STACK_LOOP)
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
def test_mixed_batches_recycle_pages(device, dtype):
    """Unequal requests batched together (portions beside single decode
    tokens) equal each request alone; the pool holds 10 pages, so later
    requests land on freed pages."""
    cfg = make_config(STACK, width=32, vocab=64, loop=STACK_LOOP)
    w = make_weights(cfg, 5)
    llm = engine(save_model(cfg, w), device, dtype, max_tokens=160)
    P = {c: tokens_for(cfg, n, 10 + i)
         for i, (c, n) in enumerate([("a", 50), ("b", 9), ("c", 33),
                                     ("d", 21), ("e", 47), ("f", 3)])}
    steps = [
        {"entries": [("a", P["a"][:18], [0, 17]), ("b", P["b"][:2], [1])]},
        {"entries": [("b", P["b"][2:3], [0]), ("a", P["a"][18:33], [14]),
                     ("c", P["c"][:30], [0, 15, 16, 29])]},
        {"entries": [("c", P["c"][30:31], [0]), ("b", P["b"][3:9], [5]),
                     ("a", P["a"][33:34], [0]), ("d", P["d"][:5], [4])],
         "end": ["b"]},
        {"entries": [("a", P["a"][34:35], [0]), ("c", P["c"][31:33], [0, 1]),
                     ("d", P["d"][5:21], [0, 15])], "end": ["c", "d"]},
        # e and f take over the pages of b, c, d
        {"entries": [("e", P["e"][:31], [15, 16, 30]), ("a", P["a"][35:36],
                                                        [0]),
                     ("f", P["f"][:3], [0, 1, 2])], "end": ["f"]},
        {"entries": [("a", P["a"][36:50], [13]), ("e", P["e"][31:32], [0])],
         "end": ["a"]},
        {"entries": [("e", P["e"][32:47], list(range(15)))], "end": ["e"]},
        # a again on recycled pages: same answers
        {"entries": [("a#2", P["a"][:50], [0, 17, 32, 49])], "end": ["a#2"]},
    ]
    used = set()
    orig = llm.scheduler.mm._allocate_fresh

    def spy(n):
        pages = orig(n)
        spy.reused |= used & set(pages)
        used.update(pages)
        return pages
    spy.reused = set()
    llm.scheduler.mm._allocate_fresh = spy
    got = run_steps(llm, steps, cfg["vocab"])
    assert spy.reused, "the schedule was meant to recycle pages"
    check_against_oracle(cfg, w, got, P, TOL[dtype])


@pytest.mark.parametrize("device,dtype", DEVICES)
def test_long_decoding(device, dtype):
    """A short prompt, then 150 tokens decoded one by one: ten pages of
    context grow under the decode path; every position checked."""
    cfg = make_config([moe(attn(heads=4, kv_heads=2, dim=8, rot_dims=8)),
                       dense(attn(heads=2, kv_heads=1, dim=16, rot_dims=6))],
                      width=24, vocab=40, loop=(0, 2, 2))
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


@pytest.mark.parametrize("dims", [(8, 4, 2), (64, 4, 4), (32, 8, 2)],
                         ids=["d8", "d64-mha", "d32"])
@pytest.mark.parametrize("device,dtype", DEVICES)
def test_planted_key_and_head_mix_stand_out(device, dtype, dims):
    """ops.talking_attention with one key whose score towers over the
    rest for ONE source head; ``talk`` is a permutation, so exactly the
    head that listens to that source returns the planted value — far
    back among hundreds of keys, at page borders, the first key, the
    query's own position, for a query inside a portion and for a decoded
    token — and a key after the query is never seen."""
    from gllm_amd import ops
    tdt = getattr(torch, dtype)
    page = 16
    D, H, G = dims
    L = 300
    g = torch.Generator().manual_seed(7)
    npages = 64
    perm = torch.randperm(npages, generator=g)[:-(-L // page)]
    bt = perm.to(torch.int32)[None].to(device)
    shift = torch.roll(torch.arange(H), 1)     # head h listens to shift[h]
    talk = torch.zeros(H, H)
    talk[torch.arange(H), shift] = 1.0
    src = 1                                     # the head that is planted
    listener = int((shift == src).nonzero()[0])
    sink = torch.randn(H, generator=g)

    def run(i, j, q_len):
        k = 0.05 * torch.randn(L, G, D, generator=g)
        v = torch.randn(L, G, D, generator=g)
        q = 0.05 * torch.randn(q_len, H, D, generator=g)
        k[j, src // (H // G), 0] = 30.0
        q[-1, :, 0] = 0.0          # only the source head answers the key
        q[-1, src, 0] = 30.0
        v[j] = 100.0
        kc, vc = _paged(k, v, perm, page, npages)
        out = ops.talking_attention(
            q.reshape(q_len, H * D).to(tdt).to(device),
            kc.to(tdt).to(device), vc.to(tdt).to(device), bt,
            torch.tensor([i + 1], dtype=torch.int32, device=device),
            torch.tensor([0, q_len], dtype=torch.int32, device=device),
            1.0, talk.to(device), sink.to(device), q_len)
        return out[-1].float().cpu().view(H, D)

    for q_len in (1, 23, 40):
        for i in (299, 271, 255, 256):
            for j, seen in [(0, True), (i, True), (i - 1, True),
                            (i - 16, True), (15, True), (16, True),
                            (i - 200, True), (i + 1, False)]:
                if j >= L:
                    continue
                o = run(i, j, q_len)
                for h in range(H):
                    if seen and h == listener:
                        assert (o[h] - 100.0).abs().max() < 1.0, \
                            (q_len, i, j, h, o[h])
                    else:
                        assert o[h].abs().max() < 10.0, (q_len, i, j, h)


@pytest.mark.parametrize("device,dtype", DEVICES)
def test_sink_takes_its_share(device, dtype):
    """Zero queries give every visible key weight 1 and the sink weight
    exp(sink_h): out = sum(v) / (n + exp(sink_h)); no sink: the mean."""
    from gllm_amd import ops
    tdt = getattr(torch, dtype)
    page, G, H, D, L = 16, 1, 2, 4, 21
    g = torch.Generator().manual_seed(8)
    kc = torch.randn(4, page, G, D, generator=g)
    vc = torch.randn(4, page, G, D, generator=g).to(tdt).float()
    bt = torch.tensor([[2, 0, 3, 1]], dtype=torch.int32, device=device)
    q = torch.zeros(L, H * D)
    talk = torch.tensor([[1.0, 0.5], [-2.0, 1.0]])
    sink = torch.tensor([0.7, -1.3])
    args = (kc.to(tdt).to(device), vc.to(tdt).to(device), bt,
            torch.tensor([L], dtype=torch.int32, device=device),
            torch.tensor([0, L], dtype=torch.int32, device=device), 0.5,
            talk.to(device))
    vs = torch.cat([vc[2], vc[0]])[:L, 0]
    for sk in (sink, None):
        out = ops.talking_attention(
            q.to(tdt).to(device), *args,
            None if sk is None else sk.to(device), L
        ).float().cpu().view(L, H, D)
        for i in (0, 1, 15, 16, 20):
            for h in range(H):
                extra = 0.0 if sk is None else math.exp(float(sk[h]))
                want = vs[:i + 1].sum(0) / (i + 1 + extra)
                tol = 1e-5 if dtype == "float32" else 2e-2
                assert (out[i, h] - want).abs().max() < tol, (sk, i, h)


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
    cfg = make_config(STACK, width=32, vocab=48, loop=STACK_LOOP,
                      softcap=30.0, logit_scale=2.0)
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
    assert checked >= 8


def test_config_and_registry():
    """The loader picks the class from config.json's architecture key;
    every layer RUN owns a KV cache entry of its own geometry."""
    from gllm_amd.config import EngineConfig
    from gllm_amd.models.loader import load_model
    cfg = make_config(STACK, width=32, vocab=48, loop=STACK_LOOP)
    d = save_model(cfg, make_weights(cfg, 15))
    model, _ = load_model(EngineConfig(model=d, dtype="float32",
                                       device="cpu"))
    assert type(model).__name__ == "GukiraxForCausalLM"
    assert model.kv_layer_shapes == [(2, 12, 12)] + \
        [(2, 16, 16), (1, 8, 8)] * 3 + [(3, 20, 20)]
    assert [r[1] for r in model.runs] == \
        [False, True, False, True, False, True, False, False]
    bad = dict(cfg, layers=[dict(STACK[0], mixer=dict(
        STACK[0]["mixer"], vdim=7))])
    with pytest.raises(ValueError):
        load_model(EngineConfig(model=save_model(bad, {}), dtype="float32",
                                device="cpu", load_format="dummy"))


# ------------------------------------------------------------ kernels vs ref
@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,G,D", [(4, 2, 16), (6, 2, 96), (8, 2, 64),
                                   (16, 4, 128), (3, 1, 20), (2, 2, 32)])
def test_talking_attention_kernels_match_reference(H, G, D, dtype):
    """Ragged batches (portions beside decode tokens), decode-only
    batches (split keys) and prompt-only batches (MFMA tiles in bf16)
    against the torch reference of the same op."""
    from gllm_amd import ops
    from gllm_amd.ops import torch_ref
    tdt = getattr(torch, dtype)
    g = torch.Generator().manual_seed(H * 100 + D)
    page, npages = 16, 96
    talk = torch.eye(H) + 0.3 * torch.randn(H, H, generator=g)
    sink = torch.randn(H, generator=g)
    for lens, qlens in [([200, 37, 1, 130], [50, 1, 1, 130]),
                        ([300, 17, 64, 65], [1, 1, 1, 1]),
                        ([257], [257]), ([129, 64], [33, 64])]:
        B = len(lens)
        kc = torch.randn(npages, page, G, D, generator=g).to(tdt)
        vc = torch.randn(npages, page, G, D, generator=g).to(tdt)
        perm = torch.randperm(npages, generator=g)
        need = [-(-n // page) for n in lens]
        bt = torch.zeros(B, max(need), dtype=torch.int32)
        at = 0
        for b, n in enumerate(need):
            bt[b, :n] = perm[at:at + n]
            at += n
        qsl = torch.tensor([0] + list(np.cumsum(qlens)), dtype=torch.int32)
        q = torch.randn(int(qsl[-1]), H * D, generator=g).to(tdt)
        sl = torch.tensor(lens, dtype=torch.int32)
        want = torch_ref.talking_attention(q, kc, vc, bt, sl, qsl, 0.2, talk,
                                           sink).float()
        got = ops.talking_attention(
            q.cuda(), kc.cuda(), vc.cuda(), bt.cuda(), sl.cuda(), qsl.cuda(),
            0.2, talk.cuda(), sink.cuda(), max(qlens)).float().cpu()
        tol = 2e-5 if dtype == "float32" else 3e-2
        assert (got - want).abs().max() < tol, (lens, qlens)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,G,D,rot", [(4, 2, 16, 8), (6, 3, 96, 32),
                                       (3, 1, 20, 20), (2, 1, 8, 0)])
def test_rotate_half_unit_norm_store_matches_reference(H, G, D, rot, dtype):
    from gllm_amd import ops
    from gllm_amd.ops import torch_ref
    tdt = getattr(torch, dtype)
    g = torch.Generator().manual_seed(D)
    T, page, npages = 45, 16, 8
    proj = torch.randn(T, (H + G) * D + 8, generator=g).to(tdt)
    pos = torch.randint(0, 5000, (T,), generator=g)
    slots = torch.randperm(page * npages, generator=g)[:T]
    freqs = torch.pow(torch.tensor(10000.0, dtype=torch.float64),
                      -2.0 * torch.arange(max(rot // 2, 1),
                                          dtype=torch.float64) / max(rot, 1))
    res = []
    for dev in ("cpu", "cuda"):
        p = proj.clone().to(dev)
        q, k = p[:, :H * D], p[:, H * D:(H + G) * D]
        kc = torch.zeros(npages, page, G, D, dtype=tdt, device=dev)
        vc = torch.zeros(npages, page, G, D, dtype=tdt, device=dev)
        fn = ops.qk_norm_rope_store if dev == "cuda" \
            else torch_ref.qk_norm_rope_store
        fn(q, k, k, None, None, pos.to(dev), slots.to(dev), freqs.to(dev),
           1.0, rot, kc, vc, H, G, D, D, 1e-6, True, True)
        res.append((q.float().cpu(), kc.float().cpu(), vc.float().cpu()))
    tol = 2e-5 if dtype == "float32" else 2e-2
    for a, b in zip(*res):
        assert (a - b).abs().max() < tol


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("width", [20, 328, 1000, 2048, 8200])
def test_gated_weight_only_layernorm_matches_reference(width, dtype):
    from gllm_amd import ops
    from gllm_amd.ops import torch_ref
    tdt = getattr(torch, dtype)
    g = torch.Generator().manual_seed(width)
    T = 37
    x = torch.randn(T, width, generator=g)
    proj = torch.randn(T, 2 * width + 8, generator=g).to(tdt)
    w1 = (1 + 0.2 * torch.randn(width, generator=g)).to(tdt)
    w2 = (1 + 0.2 * torch.randn(width, generator=g)).to(tdt)
    tol = 2e-5 if dtype == "float32" else 3e-2
    for off in (0, 8, 3):
        y, gate = proj[:, :width], proj[:, width + off:2 * width + off]
        for pre in (None, (w2, None)):
            xa, xb = x.clone(), x.clone().cuda()
            ha = torch_ref.residual_layernorm(xa, y, w1, None, 1e-6, pre,
                                              gate)
            hb = ops.residual_layernorm(
                xb, y.cuda(), w1.cuda(), None, 1e-6,
                None if pre is None else (w2.cuda(), None), gate.cuda())
            assert (xa - xb.cpu()).abs().max() < 2e-5 * 10
            if pre is not None:
                assert (ha.float() - hb.float().cpu()).abs().max() < tol
    h32 = ops.layernorm_f32(x.cuda(), w1.float().cuda(), None, 1e-6,
                            torch.float32)
    assert (h32.cpu() - torch_ref.layernorm_f32(
        x, w1.float(), None, 1e-6, torch.float32)).abs().max() < 2e-5


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_activation_kernels_match_reference(dtype):
    from gllm_amd import ops
    from gllm_amd.ops import torch_ref
    tdt = getattr(torch, dtype)
    g = torch.Generator().manual_seed(3)
    tol = 1e-5 if dtype == "float32" else 2e-2
    for n, off in [(64, 0), (36, 0), (48, 3)]:
        full = (3 * torch.randn(29, n + 8, generator=g)).to(tdt)
        x = full[:, off:off + n]
        a = ops.xielu(x.cuda(), 0.8, 1.3).float().cpu()
        b = torch_ref.xielu(x, 0.8, 1.3).float()
        assert ((a - b).abs() / (1 + b.abs())).max() < tol
        a = ops.relu2(x.cuda()).float().cpu()
        b = torch_ref.relu2(x).float()
        assert ((a - b).abs() / (1 + b.abs())).max() < tol
