"""Sudevik decoder: the engine (scheduler, paged KV / state pools, batch
builder, ops) against the plain float64 oracle in sudevik_oracle.py.

Every test builds its own small configuration and random bf16 weights,
replays token schedules through the product's trace-replay entry point
(or LLM.generate) and compares logits with the oracle run on each whole
sequence alone. CPU runs exercise the engine with the torch reference
ops; the same tests marked ``gpu`` exercise the HIP kernels in fp32
(tight tolerance) and bf16.
"""

import json
import os
import tempfile

import numpy as np
import pytest
import torch

import sudevik_oracle as oracle

DEVICES = [pytest.param("cpu", "float32", id="cpu-f32"),
           pytest.param("cuda", "float32", id="gpu-f32",
                        marks=pytest.mark.gpu),
           pytest.param("cuda", "bfloat16", id="gpu-bf16",
                        marks=pytest.mark.gpu)]
TOL = {"float32": 3e-4, "bfloat16": 8e-2}


# ------------------------------------------------------------------ models
def attn(heads=4, kv_heads=2, dim=16, vdim=8, size=7, keep=2, rot_dims=8,
         scaling=True, kv_from=None, base=10000.0, scale=0.3):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
         "scale": scale}
    if size:
        m["mask"] = {"size": size, "keep_first": keep}
    if rot_dims:
        m["rot"] = {"dims": rot_dims, "base": base}
        if scaling:
            m["rot"]["scaling"] = {"factor": 3.0, "original": 24,
                                   "fast": 8.0, "slow": 1.0}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m}


def delta(heads=4, kv_heads=2, dim=8, vdim=12, conv=3):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads,
                                       "dim": dim, "vdim": vdim,
                                       "conv": conv}}


def with_moe(layer, experts=6, top=2, ff=16):
    layer = dict(layer)
    layer["mlp"] = {"kind": "moe", "expert": {"ff": ff},
                    "router": {"experts": experts, "top": top}}
    return layer


def no_mlp(layer):
    layer = dict(layer)
    layer["mlp"] = None
    return layer


def make_config(layers, width=32, vocab=70, eps=1e-5):
    return {"architecture": "Sudevik", "layers": layers,
            "norm": {"eps": eps}, "vocab": vocab, "width": width}


def make_weights(cfg, seed):
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]
    w = {}

    def lin(name, out, inp, gain=1.0):
        w[name] = torch.randn(out, inp, generator=g) * gain / inp ** 0.5

    def norm(name, n):
        w[name] = 1.0 + 0.2 * torch.randn(n, generator=g)
        w[name + ".b"] = 0.2 * torch.randn(n, generator=g)

    w["embed"] = torch.randn(cfg["vocab"], W, generator=g)
    lin("head", cfg["vocab"], W)
    norm("final.norm", W)
    for i, layer in enumerate(cfg["layers"]):
        p = "l%d." % i
        m = layer["mixer"]
        H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        norm(p + "norm1", W)
        norm(p + "norm1b", W)
        if layer["type"] == "attention":
            lin(p + "mix.q", H * D, W, 2.0)
            w[p + "mix.q.norm"] = 1.0 + 0.3 * torch.randn(D, generator=g)
            if m.get("kv_from") is None:
                lin(p + "mix.k", G * D, W, 2.0)
                lin(p + "mix.v", G * Dv, W)
                w[p + "mix.k.norm"] = 1.0 + 0.3 * torch.randn(D, generator=g)
        else:
            lin(p + "mix.q", G * D, W, 2.0)
            lin(p + "mix.k", G * D, W, 2.0)
            lin(p + "mix.v", H * Dv, W, 2.0)
            for t, n in (("q", G * D), ("k", G * D), ("v", H * Dv)):
                w[p + "mix.%s.conv" % t] = 0.6 * torch.randn(
                    n, m["conv"], generator=g)
            lin(p + "mix.a", H, W)
            lin(p + "mix.b", H, W)
            w[p + "mix.A_log"] = torch.rand(H, generator=g) * 2 - 1.5
            w[p + "mix.dt_bias"] = torch.randn(H, generator=g)
            w[p + "mix.norm"] = 1.0 + 0.3 * torch.randn(Dv, generator=g)
        lin(p + "mix.g", H * Dv, W)
        lin(p + "mix.o", W, H * Dv)
        mlp = layer.get("mlp")
        if mlp:
            norm(p + "norm2", W)
            norm(p + "norm2b", W)
            E, ff = mlp["router"]["experts"], mlp["expert"]["ff"]
            lin(p + "mlp.router", E, W, 2.0)
            w[p + "mlp.router.b"] = 0.5 * torch.randn(E, generator=g)
            for e in range(E):
                lin(p + "mlp.e%d.gate" % e, ff, W)
                lin(p + "mlp.e%d.up" % e, ff, W)
                lin(p + "mlp.e%d.down" % e, W, ff)
    return {k: v.to(torch.bfloat16).contiguous() for k, v in w.items()}


def save_model(cfg, weights):
    from safetensors.torch import save_file
    d = tempfile.mkdtemp(prefix="sudevik_test_")
    with open(os.path.join(d, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file(weights, os.path.join(d, "model.safetensors"))
    return d


HYBRID = [with_moe(delta()), with_moe(attn()), no_mlp(attn(kv_from=1)),
          with_moe(delta(heads=2, kv_heads=2, dim=12, vdim=8, conv=4),
                   experts=4, top=1, ff=8)]


# ------------------------------------------------------------------ harness
def engine(model_dir, device, dtype, max_tokens=256, slots=4, page=16):
    from gllm_amd.entrypoints.trace_replay import build_engine
    return build_engine(model_dir, dtype, max_tokens, slots, device, page)


def run_steps(llm, steps, vocab):
    """steps: [{"entries": [(rid, tokens, want)], "end": [rid]}] ->
    {rid: {position: logits}} through trace_replay.replay."""
    from gllm_amd.entrypoints.trace_replay import replay
    out = tempfile.mkdtemp(prefix="sudevik_out_")
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
@pytest.mark.parametrize("layers", [
    [no_mlp(delta())],
    [no_mlp(delta(heads=3, kv_heads=1, dim=20, vdim=5, conv=2))],
    [no_mlp(attn())],
    [no_mlp(attn(heads=2, kv_heads=2, dim=10, vdim=24, size=0, rot_dims=0))],
    [no_mlp(attn(heads=3, kv_heads=1, dim=12, vdim=12, size=5, keep=0,
                 rot_dims=12, scaling=False))],
    [with_moe(attn(size=4, keep=1))],
    [with_moe(attn(), experts=3, top=3, ff=24)],
], ids=["delta", "delta-odd", "attn", "attn-plain", "attn-mqa", "attn-moe",
        "moe-all-experts"])
@pytest.mark.parametrize("width", [32, 36], ids=["w32", "w36"])
def test_each_mechanism_alone(layers, device, dtype, width):
    """One-layer models: each mixer / feed-forward on its own, every
    position of a whole prompt (the first tokens included). Width 36 is
    not a multiple of 8: scalar norm kernels, unaligned projection rows,
    experts on the segment loop."""
    cfg = make_config(layers, width=width)
    w = make_weights(cfg, 1)
    llm = engine(save_model(cfg, w), device, dtype)
    toks = tokens_for(cfg, 37, 2)
    got = run_steps(llm, cut("a", toks, [37]), cfg["vocab"])
    check_against_oracle(cfg, w, got, {"a": toks}, TOL[dtype])


@pytest.mark.parametrize("device,dtype", DEVICES)
def test_prefill_decode_and_portions(device, dtype):
    """Whole prompt == prompt + token-by-token decoding == portions of
    many sizes (down to two tokens and one), at every position; the
    decoded tail runs the window well past the prompt."""
    cfg = make_config(HYBRID, width=40, vocab=90)
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
    tokens) equal each request alone; the pool holds 4 state slots and
    10 pages, so later requests land on freed pages and slots."""
    cfg = make_config(HYBRID, width=32, vocab=64)
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
        # e and f take over the pages and slots of b, c, d
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
    assert llm.runner.ssm_pool.alloc.num_free == 4
    check_against_oracle(cfg, w, got, P, TOL[dtype])


@pytest.mark.parametrize("dims", [(8, 6), (64, 64)], ids=["d8", "d64"])
@pytest.mark.parametrize("device,dtype", DEVICES)
def test_window_and_kept_edges_stand_out(device, dtype, dims):
    """ops.window_attention with one planted key whose score towers over
    the rest: the output equals that key's value exactly when the key is
    visible — just inside / outside the window, the last kept token /
    the first dropped one, across page borders, far back among hundreds
    — for a query inside a prompt portion and for a decoded token."""
    from gllm_amd import ops
    tdt = getattr(torch, dtype)
    page, G, H = 16, 2, 4
    D, Dv = dims   # (64, 64) in bf16 with a portion takes the MFMA kernel
    W, keep, L = 40, 3, 300
    g = torch.Generator().manual_seed(7)
    npages = 64
    perm = torch.randperm(npages, generator=g)[:-(-L // page)]
    bt = perm.to(torch.int32)[None].to(device)

    def run(i, j, q_len):
        """Query at position i (last of a q_len portion), beacon at j."""
        k = 0.05 * torch.randn(L, G, D, generator=g)
        v = torch.randn(L, G, Dv, generator=g)
        q = 0.05 * torch.randn(q_len, H, D, generator=g)
        k[j, :, 0] = 30.0
        q[-1, :, 0] = 30.0
        v[j] = 100.0
        kc = torch.zeros(npages, page, G, D)
        vc = torch.zeros(npages, page, G, Dv)
        pos = torch.arange(L)
        kc[perm[pos // page], pos % page] = k
        vc[perm[pos // page], pos % page] = v
        out = ops.window_attention(
            q.reshape(q_len, H * D).to(tdt).to(device), None,
            kc.to(tdt).to(device), vc.to(tdt).to(device), bt,
            torch.tensor([i + 1], dtype=torch.int32, device=device),
            torch.tensor([0, q_len], dtype=torch.int32, device=device),
            1.0, W, keep, True, q_len)
        return out[-1].float().cpu()

    for q_len in (1, 23):
        for i in (299, 271, 255, 256):
            cases = [(i - W + 1, True), (i - W, False), (keep - 1, True),
                     (keep, False), (0, True), (i, True), (i - 1, True),
                     (i - 16, True), (i - W - 100, False)]
            for j, seen in cases:
                o = run(i, j, q_len)
                if seen:
                    assert (o - 100.0).abs().max() < 1.0, (q_len, i, j, o)
                else:
                    assert o.abs().max() < 10.0, (q_len, i, j, o)
    # plain causal (no window): a key hundreds back is seen
    k = 0.05 * torch.randn(L, G, D, generator=g)
    v = torch.randn(L, G, Dv, generator=g)
    k[5, :, 0] = 30.0
    v[5] = 100.0
    q = torch.zeros(1, H, D)
    q[0, :, 0] = 30.0
    kc = torch.zeros(npages, page, G, D)
    vc = torch.zeros(npages, page, G, Dv)
    pos = torch.arange(L)
    kc[perm[pos // page], pos % page] = k
    vc[perm[pos // page], pos % page] = v
    out = ops.window_attention(
        q.reshape(1, H * D).to(tdt).to(device), None, kc.to(tdt).to(device),
        vc.to(tdt).to(device), bt,
        torch.tensor([L], dtype=torch.int32, device=device),
        torch.tensor([0, 1], dtype=torch.int32, device=device),
        1.0, 0, 0, True)
    assert (out.float().cpu() - 100.0).abs().max() < 1.0


@pytest.mark.parametrize("device,dtype", DEVICES)
def test_sink_takes_its_share(device, dtype):
    """Zero queries give every visible key and the sink the same weight:
    out = sum(v) / (n + 1); without the sink it is the plain mean."""
    from gllm_amd import ops
    tdt = getattr(torch, dtype)
    page, G, H, D, Dv, L = 16, 1, 2, 4, 3, 21
    g = torch.Generator().manual_seed(8)
    kc = torch.randn(4, page, G, D, generator=g)
    vc = torch.randn(4, page, G, Dv, generator=g).to(tdt).float()
    bt = torch.tensor([[2, 0, 3, 1]], dtype=torch.int32, device=device)
    q = torch.zeros(L, H * D)
    args = (kc.to(tdt).to(device), vc.to(tdt).to(device), bt,
            torch.tensor([L], dtype=torch.int32, device=device),
            torch.tensor([0, L], dtype=torch.int32, device=device), 0.5)
    vs = torch.cat([vc[2], vc[0]])[:L, 0]
    for sink in (True, False):
        out = ops.window_attention(q.to(tdt).to(device), None, *args, 0, 0,
                                   sink).float().cpu().view(L, H, Dv)
        for i in (0, 1, 15, 16, 20):
            want = vs[:i + 1].sum(0) / (i + 1 + (1 if sink else 0))
            tol = 1e-5 if dtype == "float32" else 2e-2
            assert (out[i, 0] - want).abs().max() < tol, (sink, i)


@pytest.mark.parametrize("device,dtype", DEVICES)
def test_far_state_survives_long_decoding(device, dtype):
    """A delta-only model decoded token by token for 100 steps after a
    short prompt: the state carries the early tokens all the way."""
    cfg = make_config([no_mlp(delta(conv=4)), no_mlp(delta(
        heads=2, kv_heads=1, dim=16, vdim=16, conv=2))], width=24, vocab=40)
    w = make_weights(cfg, 9)
    for i in range(2):  # slow decay, or 100 random steps forget the start
        w["l%d.mix.A_log" % i] = torch.full_like(w["l%d.mix.A_log" % i], -7.0)
        w["l%d.mix.dt_bias" % i] = torch.full_like(
            w["l%d.mix.dt_bias" % i], -1.0)
    llm = engine(save_model(cfg, w), device, dtype)
    toks = tokens_for(cfg, 110, 11)
    steps = cut("a", toks, [10] + [1] * 100, want_all=False)
    got = run_steps(llm, steps, cfg["vocab"])
    check_against_oracle(cfg, w, got, {"a": toks}, TOL[dtype])
    # and the early tokens matter: another start gives another end
    other = list(toks)
    other[0] = (other[0] + 1) % cfg["vocab"]
    a = oracle.forward(cfg, w, toks)[-1].numpy()
    b = oracle.forward(cfg, w, other)[-1].numpy()
    assert rel_err(b.astype(np.float32), a) > 0.05


@pytest.mark.parametrize("device,dtype", DEVICES)
def test_window_passes_over_decoded_tokens(device, dtype):
    """Attention-only stack with a short window and kept tokens, decoded
    far past the window: every decoded position against the oracle."""
    cfg = make_config([with_moe(attn(size=9, keep=3, dim=16, vdim=16,
                                     rot_dims=16)),
                       no_mlp(attn(size=9, keep=3, dim=16, vdim=16,
                                   rot_dims=16, kv_from=0)),
                       no_mlp(attn(heads=2, kv_heads=1, dim=8, vdim=4,
                                   size=17, keep=0, rot_dims=4))],
                      width=32, vocab=50)
    w = make_weights(cfg, 12)
    llm = engine(save_model(cfg, w), device, dtype)
    toks = tokens_for(cfg, 70, 13)
    steps = cut("a", toks, [6] + [1] * 64)
    got = run_steps(llm, steps, cfg["vocab"])
    check_against_oracle(cfg, w, got, {"a": toks}, TOL[dtype])


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
    cfg = make_config(HYBRID, width=32, vocab=48)
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
    per-layer KV / state geometry follows the layer list."""
    from gllm_amd.config import EngineConfig
    from gllm_amd.models.loader import load_model
    from gllm_amd.parallel import init_distributed
    cfg = make_config(HYBRID)
    d = save_model(cfg, make_weights(cfg, 15))
    ec = EngineConfig(model=d, dtype="float32", device="cpu")
    init_distributed(ec)
    model, _ = load_model(ec, "cpu")
    assert type(model).__name__ == "SudevikForCausalLM"
    assert model.kv_layer_shapes == [(2, 16, 8)]       # layer 2 borrows
    assert [(s.conv_dim, s.conv_kernel, s.head_k_dim, s.head_v_dim)
            for s in model.ssm_spec.layers] == [(80, 3, 8, 12),
                                                (64, 4, 12, 8)]
    with pytest.raises(KeyError):
        model.load_weights([("l0.mix.nonsense", torch.zeros(1))])


@pytest.mark.gpu
@pytest.mark.parametrize("D,Dv,dtype", [
    (64, 64, "bfloat16"), (128, 128, "bfloat16"), (64, 64, "float32"),
    (24, 40, "bfloat16"), (16, 8, "float32"), (128, 64, "bfloat16"),
    (32, 320, "float32"), (7, 3, "float32")])
@pytest.mark.parametrize("window,keep", [(50, 3), (0, 0), (130, 70),
                                         (10, 40)])
def test_window_attention_kernels_match_reference(D, Dv, dtype, window,
                                                  keep):
    """Both GPU kernels (MFMA tiles for bf16 D == Dv in {64, 128} when a
    portion is in the batch, the generic kernel otherwise) against the
    torch reference of the same op on a ragged batch: portions with and
    without a past beside single decode tokens, shuffled pages, gate."""
    from gllm_amd import ops
    from gllm_amd.ops import torch_ref
    tdt = getattr(torch, dtype)
    g = torch.Generator().manual_seed(D + Dv + window)
    page, G, H = 16, 2, 8
    geo = [(0, 200), (37, 1), (130, 77), (300, 1), (5, 2), (63, 129)]
    lens = [p + n for p, n in geo]
    npages = sum(-(-L // page) for L in lens) + 3
    perm = torch.randperm(npages, generator=g).tolist()
    maxp = max(-(-L // page) for L in lens)
    bt = torch.zeros(len(geo), maxp, dtype=torch.int32)
    for b, L in enumerate(lens):
        n = -(-L // page)
        bt[b, :n] = torch.tensor([perm.pop() for _ in range(n)])
    kc = torch.randn(npages, page, G, D, generator=g).to(tdt)
    vc = torch.randn(npages, page, G, Dv, generator=g).to(tdt)
    T = sum(n for _, n in geo)
    q = (torch.randn(T, H * D, generator=g) * 0.5).to(tdt)
    gate = torch.randn(T, H * Dv, generator=g).to(tdt)
    qsl = torch.tensor([0] + list(np.cumsum([n for _, n in geo])),
                       dtype=torch.int32)
    sl = torch.tensor(lens, dtype=torch.int32)
    scale = D ** -0.5
    for use_gate in (True, False):
        for sink in (True, False):
            gt = gate if use_gate else None
            want = torch_ref.window_attention(
                q.float(), None if gt is None else gt.float(), kc.float(),
                vc.float(), bt, sl, qsl, scale, window, keep, sink)
            got = ops.window_attention(
                q.cuda(), None if gt is None else gt.cuda(), kc.cuda(),
                vc.cuda(), bt.cuda(), sl.cuda(), qsl.cuda(), scale,
                window, keep, sink, 200).float().cpu()
            tol = 2e-2 if dtype == "bfloat16" else 2e-5
            err = (got - want).abs().max().item()
            assert err < tol, (use_gate, sink, err)
            # decode-only batch: one new token per sequence (bf16 with
            # an instantiated geometry takes the split-KV kernels)
            last = qsl[1:].long() - 1
            ar = torch.arange(len(geo) + 1, dtype=torch.int32)
            got = ops.window_attention(
                q[last].cuda(), None if gt is None else gt[last].cuda(),
                kc.cuda(), vc.cuda(), bt.cuda(), sl.cuda(), ar.cuda(),
                scale, window, keep, sink, 1).float().cpu()
            err = (got - want[last]).abs().max().item()
            assert err < tol, ("decode", use_gate, sink, err)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("off", [3, 8], ids=["unaligned", "aligned"])
@pytest.mark.parametrize("H,G,Dk,Dv,taps", [
    (4, 2, 128, 128, 4), (3, 1, 20, 5, 2), (2, 2, 64, 96, 3),
    (8, 4, 32, 16, 1), (2, 1, 200, 72, 8), (4, 4, 16, 64, 5)])
def test_delta_rule_kernels_match_reference(H, G, Dk, Dv, taps, dtype, off):
    """causal_conv_silu + delta_rule_varlen + rms_gate on the GPU against
    the torch reference of the same ops: ragged batch (fresh portions,
    continued portions, decode tokens), state slots out of order."""
    from gllm_amd import ops
    from gllm_amd.ops import gdn_ref
    tdt = getattr(torch, dtype)
    g = torch.Generator().manual_seed(H * Dk + Dv + taps)
    geo = [(False, 70), (True, 1), (True, 9), (False, 2), (True, 1)]
    slots = torch.tensor([3, 0, 5, 1, 4])
    n_slots = 7
    T = sum(n for _, n in geo)
    C = 2 * G * Dk + H * Dv
    qsl = torch.tensor([0] + list(np.cumsum([n for _, n in geo])),
                       dtype=torch.int32)
    init = torch.tensor([int(i) for i, _ in geo], dtype=torch.int32)
    # a column slice of a wider buffer; the aligned one takes the 16 B
    # vector kernels where the shapes allow
    x = torch.randn(T, C + 16, generator=g).to(tdt)[:, off:off + C]
    w = (torch.randn(C, taps, generator=g) * 0.5).to(tdt)
    cs = torch.randn(n_slots, C, max(taps - 1, 1), generator=g).to(tdt)
    st = torch.randn(n_slots, H, Dk, Dv, generator=g) * 0.3
    ab = torch.randn(T, 2 * H, generator=g).to(tdt)
    A_log = torch.rand(H, generator=g) * 2 - 1.5
    dtb = torch.randn(H, generator=g)
    z = torch.randn(T, H * Dv, generator=g).to(tdt)
    nw = (1 + 0.2 * torch.randn(Dv, generator=g)).to(tdt)

    def run(dev, mql=0):
        cs_d, st_d = cs.clone().to(dev), st.clone().to(dev)
        conv = ops.causal_conv_silu(x.to(dev), w.to(dev), cs_d,
                                    slots.to(dev), init.to(dev),
                                    qsl.to(dev))
        gk = G * Dk
        abd = ab.to(dev)
        o = ops.delta_rule_varlen(
            conv[:, :gk], conv[:, gk:2 * gk], conv[:, 2 * gk:],
            abd[:, :H], abd[:, H:], A_log.to(dev), dtb.to(dev), st_d,
            slots.to(dev), init.to(dev), qsl.to(dev), Dk ** -0.5, mql)
        out = ops.rms_gate(o, z.to(dev), nw.to(dev), H, 1e-5, tdt)
        return (conv.float().cpu(), o.cpu(), out.float().cpu(),
                cs_d.float().cpu(), st_d.cpu())

    want = run("cpu")
    tol = 3e-2 if dtype == "bfloat16" else 1e-4
    # 0: LDS-tiled recurrence (batches with portions); 1: the register
    # form decode-only batches take (valid for any portion length)
    for mql in (0, 1):
        got = run("cuda", mql)
        for name, a, b in zip(("conv", "o", "out", "conv_state", "state"),
                              want, got):
            scale = max(1.0, a.abs().max().item())
            assert (a - b).abs().max().item() < tol * scale, (name, mql)
        # untouched slots stay as they were
        assert torch.equal(got[4][2], st[2])
        assert torch.equal(got[4][6], st[6])


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("width", [20, 32, 1000, 2048, 8200])
def test_layernorm_kernels_match_reference(width, dtype):
    """layernorm_f32 / residual_layernorm on the GPU (scalar, 8-wide LDS
    and wave-per-row variants by width) against the torch reference."""
    from gllm_amd import ops
    from gllm_amd.ops import torch_ref
    tdt = getattr(torch, dtype)
    g = torch.Generator().manual_seed(width)
    rows = 37
    x = torch.randn(rows, width, generator=g) * 3
    y = torch.randn(rows, width + 8, generator=g).to(tdt)[:, :width]
    w1, b1, w2, b2 = [(torch.randn(width, generator=g) * 0.3 + s).to(tdt)
                      for s in (1, 0, 1, 0)]
    tol = 3e-2 if dtype == "bfloat16" else 1e-5
    want = torch_ref.layernorm_f32(x, w1, b1, 1e-5, tdt).float()
    got = ops.layernorm_f32(x.cuda(), w1.cuda(), b1.cuda(), 1e-5,
                            tdt).float().cpu()
    assert (got - want).abs().max() < tol
    for pre in (None, (w2, b2)):
        xc, xg = x.clone(), x.clone().cuda()
        hw = torch_ref.residual_layernorm(xc, y, w1, b1, 1e-5, pre)
        hg = ops.residual_layernorm(
            xg, y.cuda(), w1.cuda(), b1.cuda(), 1e-5,
            None if pre is None else (w2.cuda(), b2.cuda()))
        assert (xg.cpu() - xc).abs().max() < 1e-5 * 10
        if pre is not None:
            assert (hg.float().cpu() - hw.float()).abs().max() < tol


@pytest.mark.parametrize("device,dtype", DEVICES)
def test_prefix_cache_hit_restores_state(device, dtype):
    """A second prompt that shares two full pages with an earlier one
    re-uses the cached KV pages and the recurrent-state snapshot taken at
    that page boundary; its greedy continuation still matches the oracle."""
    from gllm_amd.config import EngineConfig
    from gllm_amd.engine.llm import LLM
    from gllm_amd.sequence import SamplingParams
    cfg = make_config(HYBRID, width=32, vocab=48)
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
