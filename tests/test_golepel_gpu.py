"""Golepel on the GPU: each mechanism's kernels alone against the plain functions of tests/plain, then the model through
the step function, the cache and the generation entry point, in float32 and bfloat16."""
import pytest
import torch

from trapetum_amd.cache import ModelCache
from trapetum_amd.engine.batch import StepContext
from trapetum_amd.engine.runtime import Runtime
from trapetum_amd.registry import build_part

from . import golepel_tiny as gt
from .plain import golepel_plain as plain
from .tiny import random_tokens, rel_l2

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = {"float32": 2e-5, "bfloat16": gt.Rounded(4e-2)}
PART_TOL = {torch.float32: 3e-6, torch.bfloat16: 1e-2}


def rnd(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


@pytest.fixture(scope="module", params=["float32", "bfloat16"])
def rt(request):
    return Runtime(dtype=request.param, device=DEV)


def stored(rt, t):
    """A tensor as a model folder stores it (bf16), on the device and widened for the plain functions."""
    b = t.to(torch.bfloat16)
    return b.to(DEV), b.double()


def acts(rt, t):
    """Rows in the activation dtype, on the device and as the plain functions see them."""
    a = t.to(rt.dtype)
    return a.to(DEV), a.double()


# ---- each mechanism alone -----------------------------------------------------------------------------------------------
@pytest.mark.parametrize("m,d,groups", [(5, 96, 3), (300, 512, 2), (3, 50, 1), (200, 2304, 4), (7, 9000, 3)])
def test_group_norm(rt, m, d, groups):
    tol = PART_TOL[rt.dtype]
    norm = build_part("norm", ("rms_norm", {"size": d, "eps": 1e-5, "groups": groups, "tensor": ""}))
    w_dev, w = stored(rt, 1.0 + rnd(d, seed=1, scale=0.3))
    norm.bind({"": w_dev}, rt)
    x = rnd(m, d, seed=2)
    ctx = type("C", (), {"ops": rt.ops, "dtype": rt.dtype})()
    assert rel_l2(norm.forward(ctx, x.to(DEV)), plain.group_rms_norm(x.double(), w, 1e-5, groups)) < tol
    # the stream takes the normed rows, and the next norm of the sum comes back, from one kernel
    rows_dev, rows = acts(rt, rnd(m, d, seed=3))
    stream = x.to(DEV).clone()
    nxt = rt.ops.add_rms_norm(stream, rows_dev, norm.gain, 1e-5, norm.gain, 1e-5, rt.dtype, groups=groups)
    want = x.double() + plain.group_rms_norm(rows, w, 1e-5, groups)
    assert rel_l2(stream, want) < 3e-6
    assert rel_l2(nxt, plain.group_rms_norm(want, w, 1e-5, groups)) < tol


@pytest.mark.parametrize("taps,d", [(4, 96), (2, 700), (1, 50), (7, 33)])
def test_causal_conv_with_state(rt, taps, d):
    conv = build_part("conv", ("causal_conv", {"size": d, "taps": taps, "tensor": ""}))
    w_dev, w = stored(rt, rnd(d, taps, seed=4, scale=0.5))
    conv.bind({"": w_dev}, rt)
    spec = conv.state_spec()
    assert (spec is None) == (taps == 1)
    cache = ModelCache([None], 512, 512, 4, 16, rt.dtype, rt.device, entry_states=[{"c": spec}] if spec else None)
    seqs = {0: rnd(40, d, seed=5), 1: rnd(9, d, seed=6), 2: rnd(23, d, seed=7)}
    want = {i: x.double() + plain.causal_conv(x.double(), w) for i, x in seqs.items()}
    slots = {i: cache.acquire() for i in seqs}
    got = {i: [] for i in seqs}
    done = {i: 0 for i in seqs}
    # steps of unequal portions (one shorter than the taps reach), then single rows, then a portion again
    for counts in ({0: 5, 1: 1, 2: 2}, {0: 1, 1: 1, 2: 1}, {0: 1, 2: 1}, {0: 20, 1: 7, 2: 3}, {0: 13, 2: 16}):
        ids = sorted(counts)
        starts = [cache.length(slots[i]) for i in ids]
        for i in ids:
            cache.grow(slots[i], counts[i])
        ctx = StepContext(rt, cache, [slots[i] for i in ids], [counts[i] for i in ids], starts, [])
        ctx.entry = ctx.cache_owner = 0
        x = torch.cat([seqs[i][done[i]:done[i] + counts[i]] for i in ids]).to(DEV)
        out = conv.forward(ctx, x, cache.entry_state(0, "c") if spec else None)
        at = 0
        for i in ids:
            got[i].append(out[at:at + counts[i]])
            at += counts[i]
            done[i] += counts[i]
    for i in seqs:
        assert done[i] == seqs[i].shape[0]
        assert rel_l2(torch.cat(got[i]), want[i]) < PART_TOL[rt.dtype], i


def latent_part(rt, H, dn, dr, dv, R, rot, own=True, seed=0, scale=0.3):
    part = build_part("mixer", ("latent_attention", dict(
        hidden_size=72, num_heads=H, nope_dim=dn, rope_dim=dr, value_dim=dv, latent_rank=R, scale=scale, latent_eps=1e-5,
        own_latent=own, position=("rope", {"rotary_dim": rot, "theta": 300.0}) if rot else ("none", {}))))
    T = {"q": rnd(H * (dn + dr), 72, seed=seed + 1, scale=0.2), "uk": rnd(H * dn, R, seed=seed + 2, scale=0.3),
         "uv": rnd(H * dv, R, seed=seed + 3, scale=0.3), "o": rnd(72, H * dv, seed=seed + 4, scale=0.2)}
    if own:
        T["dkv"] = rnd(R + dr, 72, seed=seed + 5, scale=0.2)
        T["dkv.norm"] = 1.0 + rnd(R, seed=seed + 6, scale=0.3)
    dev, wide = {}, {}
    for k, v in T.items():
        dev[k], wide["mix." + k] = stored(rt, v)
    part.bind(dev, rt)
    sizes = {"heads": H, "dim": dn, "rot_dim": dr, "vdim": dv, "kv_rank": R, "scale": scale, "rot": {"base": 300.0, "dims": rot}}
    return part, wide, sizes


@pytest.mark.parametrize("H,dn,dr,dv,R,rot", [(3, 16, 16, 24, 32, 8), (1, 12, 6, 10, 20, 0), (20, 8, 8, 16, 24, 8),
                                              (4, 32, 32, 32, 96, 32), (2, 24, 16, 8, 280, 16),
                                              # cached rows of every multiple of 16 elements the matrix-core attention takes
                                              (4, 16, 16, 16, 80, 16), (2, 16, 32, 16, 80, 32), (3, 8, 16, 8, 128, 16),
                                              (5, 8, 16, 8, 144, 8), (2, 8, 16, 8, 160, 16), (16, 8, 32, 8, 160, 32),
                                              (2, 8, 16, 8, 192, 16), (7, 8, 16, 8, 208, 16), (1, 8, 16, 8, 224, 16),
                                              (16, 8, 64, 8, 192, 64), (17, 8, 16, 8, 48, 16)])
def test_latent_attention_part(rt, H, dn, dr, dv, R, rot):
    """The mixer alone: a prompt, single tokens, a portion; then a second part without a down-projection on the same cache."""
    tol = PART_TOL[rt.dtype] * (3 if rt.dtype == torch.float32 else 1.5)
    part, W, sizes = latent_part(rt, H, dn, dr, dv, R, rot)
    reader, W2, _ = latent_part(rt, H, dn, dr, dv, R, rot, own=False, seed=50)
    n = 75
    x_dev, x = acts(rt, rnd(n, 72, seed=9))
    pos = torch.arange(n)
    lat = plain.latent_keys(x, W["mix.dkv"], W["mix.dkv.norm"], 1e-5, R, pos, sizes["rot"])
    want = plain.latent_attention(x, W, "mix.", sizes, pos, lat)
    want2 = plain.latent_attention(x, W2, "mix.", sizes, pos, lat)
    cache = ModelCache([part.cache_spec(), None], 256, 256, 2, 16, rt.dtype, rt.device)
    s = cache.acquire()
    got, got2, at = [], [], 0
    for count in (33, 1, 1, 1, 30, 2, 1, 6):
        start = cache.length(s)
        cache.grow(s, count)
        ctx = StepContext(rt, cache, [s], [count], [start], [])
        ctx.mark_shared([0])
        ctx.entry = ctx.cache_owner = 0
        got.append(rt.ops.rows(part.forward(ctx, x_dev[at:at + count], cache.site(0)), rt.dtype))
        ctx.entry = 1
        got2.append(rt.ops.rows(reader.forward(ctx, x_dev[at:at + count], cache.site(0)), rt.dtype))
        ctx.finish()
        at += count
    assert at == n
    assert rel_l2(torch.cat(got), want) < tol
    assert rel_l2(torch.cat(got2), want2) < tol


def test_latent_attention_long_context(rt):
    """Beyond 1,536 keys the decode attention takes the heads in groups of 8: a prompt of 1,600 tokens, then single tokens."""
    H, dn, dr, dv, R, rot = 8, 16, 16, 16, 48, 16
    part, W, sizes = latent_part(rt, H, dn, dr, dv, R, rot, scale=0.6)
    n, first = 1640, 1600
    x_dev, x = acts(rt, rnd(n, 72, seed=12))
    pos = torch.arange(n)
    lat = plain.latent_keys(x, W["mix.dkv"], W["mix.dkv.norm"], 1e-5, R, pos, sizes["rot"])
    want = plain.latent_attention(x, W, "mix.", sizes, pos, lat)
    cache = ModelCache([part.cache_spec()], 2048, 2048, 2, 64, rt.dtype, rt.device)
    s = cache.acquire()
    got, at = [], 0
    for count in [first] + [1] * (n - first):
        start = cache.length(s)
        cache.grow(s, count)
        ctx = StepContext(rt, cache, [s], [count], [start], [])
        ctx.entry = ctx.cache_owner = 0
        got.append(rt.ops.rows(part.forward(ctx, x_dev[at:at + count], cache.site(0)), rt.dtype))
        at += count
    got = torch.cat(got)
    # float32 angles of a thousand radians and more are rounded to about 1e-4 of a radian: some 1e-5 of the output
    tol = 5e-5 if rt.dtype == torch.float32 else 3e-2
    assert rel_l2(got[:first], want[:first]) < tol
    for i in range(first, n):
        assert rel_l2(got[i], want[i]) < 2 * tol, i


@pytest.mark.parametrize("m,h,n,k,lead", [(5, 3, 32, 16, 16), (100, 4, 24, 40, 8), (700, 2, 200, 72, 0), (9, 5, 7, 12, 6), (600, 3, 50, 24, 16)])
def test_head_linear(rt, m, h, n, k, lead):
    """Per-head products on views of wider rows: each head's `k` elements follow `lead` others, and the output lands
    behind `lead` elements of each head of a wider row as well."""
    x = rnd(m, h, lead + k, seed=70).to(rt.dtype).to(DEV)
    w = rnd(h, n, k, seed=71, scale=0.3).to(rt.dtype).to(DEV)
    want = torch.einsum("mhk,hnk->mhn", x[:, :, lead:].double().cpu(), w.double().cpu())
    got = rt.ops.head_linear(x[:, :, lead:], w)
    assert got.is_contiguous() and rel_l2(got, want) < PART_TOL[rt.dtype]
    wide = torch.full((m, h, lead + n), 7.0, dtype=rt.dtype, device=DEV)
    rt.ops.head_linear(x[:, :, lead:], w, wide[:, :, lead:])
    assert rel_l2(wide[:, :, lead:], want) < PART_TOL[rt.dtype]
    assert bool((wide[:, :, :lead] == 7.0).all())


@pytest.mark.parametrize("H", [4, 24])              # 24: more heads than a decode launch takes, run in groups
@pytest.mark.parametrize("page,counts", [(16, (15, 1, 1, 1, 31, 2, 1, 40, 1, 1, 1, 1, 1, 2)), (64, (64, 1, 30, 1, 1, 1, 1, 1))])
def test_latent_attention_sharp_scores(rt, page, counts, H):
    """Scores scaled until a softmax picks single keys, wherever they lie: a key lost or read one row off, at a page's
    border or far back, then changes a row's output by about as much as the output itself."""
    dn, dr, dv, R, rot = 16, 16, 16, 48, 16
    part, W, sizes = latent_part(rt, H, dn, dr, dv, R, rot, scale=2.5)
    n = sum(counts)
    x_dev, x = acts(rt, rnd(n, 72, seed=10))
    pos = torch.arange(n)
    lat = plain.latent_keys(x, W["mix.dkv"], W["mix.dkv.norm"], 1e-5, R, pos, sizes["rot"])
    want = plain.latent_attention(x, W, "mix.", sizes, pos, lat)
    cache = ModelCache([part.cache_spec()], 256, 256, 2, page, rt.dtype, rt.device)
    cache.release(cache.acquire())
    s = cache.acquire()
    got, at = [], 0
    for count in counts:
        start = cache.length(s)
        cache.grow(s, count)
        ctx = StepContext(rt, cache, [s], [count], [start], [])
        ctx.entry = ctx.cache_owner = 0
        got.append(rt.ops.rows(part.forward(ctx, x_dev[at:at + count], cache.site(0)), rt.dtype))
        at += count
    got = torch.cat(got)
    errs = [rel_l2(got[i], want[i]) for i in range(n)]
    assert max(errs) < (2e-4 if rt.dtype == torch.float32 else 0.25), (errs.index(max(errs)), max(errs))
    assert sorted(errs)[n // 2] < (2e-5 if rt.dtype == torch.float32 else 4e-2)


@pytest.mark.parametrize("m,d,f,e,top,limit", [(1, 64, 40, 5, 3, 0.8), (9, 50, 18, 2, 2, 0.5), (150, 96, 70, 16, 2, 1.5),
                                               (70, 128, 33, 9, 1, 2.0), (300, 72, 24, 130, 4, 1.0), (650, 136, 200, 3, 2, 1.2), (5, 64, 1024, 3, 2, 1.0),
                                               (700, 128, 192, 3, 2, 1.0), (530, 192, 320, 2, 2, 0.9), (900, 64, 64, 7, 1, 1.5)])
def test_routed_experts(rt, m, d, f, e, top, limit):
    part = build_part("feed_forward", ("routed_experts", dict(hidden_size=d, intermediate_size=f, n_experts=e, top=top, limit=limit)))
    dev, W = {}, {}
    dev["router"], W["router"] = stored(rt, rnd(e, d, seed=20, scale=0.4))
    for k in range(e):
        for name, shape in (("gate", (f, d)), ("up", (f, d)), ("down", (d, f))):
            dev[f"e{k}.{name}"], W[f"e{k}.{name}"] = stored(rt, rnd(*shape, seed=21 + 3 * k + len(name), scale=0.3))
    part.bind(dev, rt)
    x_dev, x = acts(rt, rnd(m, d, seed=19))
    ctx = type("C", (), {"ops": rt.ops, "dtype": rt.dtype})()
    mlp = {"router": {"experts": e, "top": top}, "expert": {"limit": limit}}
    idx, val = plain.route(x, W["router"], top)
    logits = rt.ops.linear(x_dev, part.w_router, torch.float32)
    chosen, weights = rt.ops.route_top(logits, top)
    assert torch.equal(chosen.cpu().long(), idx) and rel_l2(weights, val) < 1e-5
    got = part.forward(ctx, x_dev)
    assert got.dtype == torch.float32
    assert rel_l2(got, plain.moe_ff(x, W, "", mlp)) < PART_TOL[rt.dtype]


def test_route_top_takes_the_smaller_index_of_equals():
    rt = Runtime(dtype="float32", device=DEV)
    z = torch.zeros(3, 70)
    z[0, [5, 69, 64]] = 2.0
    z[1, [0, 1]] = 1.0
    chosen, w = rt.ops.route_top(z.to(DEV), 2)
    assert chosen.cpu().tolist() == [[5, 64], [0, 1], [0, 1]]
    assert abs(float(w[2, 0]) - 1 / 70) < 1e-7


# ---- the model ------------------------------------------------------------------------------------------------------------
@pytest.fixture(scope="module", params=[("P", "float32"), ("P", "bfloat16"), ("Q", "float32"), ("Q", "bfloat16")],
                ids=lambda p: f"{p[0]}-{p[1]}")
def m(request, tmp_path_factory):
    from .gpu_engine import load_gpu_model
    which, dtype = request.param
    folder = gt.make_folder(tmp_path_factory.mktemp("g"), which)
    model, cfg = load_gpu_model(folder, dtype)
    pcfg, pw = plain.read_folder(folder)
    return model, cfg, pcfg, pw, TOL[dtype]


@pytest.fixture(scope="module")
def sharp(tmp_path_factory):
    from .gpu_engine import load_gpu_model
    folder = gt.make_folder(tmp_path_factory.mktemp("g"), "S")
    model, cfg = load_gpu_model(folder, "float32")
    pcfg, pw = plain.read_folder(folder)
    return model, cfg, pcfg, pw, 4e-3


def test_whole_and_token_by_token(m):
    gt.whole_and_token_by_token(m)


def test_prompt_then_long_decode(m):
    gt.prompt_then_decode(m, n=400, tail=300)


def test_portions(m):
    gt.portions(m)


def test_unequal_batches_and_reuse(m):
    gt.unequal_batches_and_reuse(m)


def test_slot_after_a_longer_sequence(m):
    gt.slot_after_a_longer_sequence(m)


def test_sharp_scores_far_keys(sharp):
    gt.sharp_scores_far_keys(sharp, n=420, page=64)
    gt.sharp_scores_far_keys(sharp, n=150, page=16)


def test_layers_one_by_one(m):
    """The residual stream after every layer, as the debug dump's l2 of the stage `layer_out` reports it."""
    model, cfg, pcfg, pw, tol = m
    toks = random_tokens(21, cfg.vocab_size, 81)
    want = []
    plain.forward(pcfg, pw, toks, want)
    seen = []
    cache = model.new_cache(max_tokens=64, page_size=16)
    s = cache.acquire()
    counts, starts, rows, tok = model.prepare(cache, [s], toks, counts=[len(toks)], want=[len(toks) - 1])    # reserves the pages first
    ctx = StepContext(model.rt, cache, [s], counts, starts, rows)
    ctx.dump = lambda stage, x: seen.append(x.clone()) if stage == "layer_out" else None
    model.run(ctx, tok)
    assert len(seen) == len(want)
    for i, (a, b) in enumerate(zip(seen, want)):
        gt.rows_close(a, b, tol, i)


@pytest.mark.parametrize("which,dtype", [("P", "float32"), ("Q", "float32"), ("P", "bfloat16")])
def test_greedy_generation_through_the_entry_point(which, dtype, tmp_path):
    from trapetum_amd import load_model
    folder = gt.make_folder(tmp_path, which)
    pcfg, pw = plain.read_folder(folder)
    prompts = [random_tokens(n, pcfg["vocab"], 90 + n) for n in (7, 1, 19, 4, 33)]
    engine = load_model(folder, dtype=dtype, max_tokens_in_cache=64 * 3, max_batch=3)      # graphs on; slots are used again
    got = engine.generate(prompts, max_tokens=12, stop_ids=())
    assert [len(g) for g in got] == [12] * len(prompts)
    if dtype == "float32":
        assert got == [plain.greedy_generate(pcfg, pw, p, 12) for p in prompts]
    again = engine.generate(prompts[::-1], max_tokens=12, stop_ids=())       # replayed graphs, other slots
    assert again == got[::-1]
    assert engine.cache.live_slots() == []


# ---- the programs a user runs ------------------------------------------------------------------------------------------------
def test_command_line_and_trace_runner(tmp_path):
    """`python -m trapetum_amd random | run | generate` and bin/trace_run on a Golepel folder: the model class comes from
    config.json, the ids and logits are the plain implementation's."""
    import json
    import os
    import subprocess
    import sys

    import numpy as np

    from . import trace_schedules as ts
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

    def run(cmd, **kw):
        p = subprocess.run(cmd, cwd=root, capture_output=True, text=True, timeout=300, **kw)
        assert p.returncode == 0, p.stderr[-2000:]
        return p.stdout
    cfg, init = gt.CONFIGS["P"]
    config = tmp_path / "config.json"
    config.write_text(json.dumps(cfg))
    folder = tmp_path / "model"
    module = [sys.executable, "-m", "trapetum_amd"]
    assert "wrote" in run(module + ["random", "--config", str(config), "--out", str(folder), "--seed", str(init["seed"]),
                                    "--sigma", str(init["sigma"]), "--sigma-norm", str(init["sigma_norm"])])
    pcfg, pw = plain.read_folder(str(folder))
    prompts = [random_tokens(n, pcfg["vocab"], 95 + n) for n in (6, 13)]
    want = [plain.greedy_generate(pcfg, pw, p, 7) for p in prompts]
    out = run(module + ["run", str(folder), "--prompt-ids", ",".join(map(str, prompts[0])), "--max-tokens", "7", "--dtype", "float32"])
    assert out.strip() == f"continuation ids: {want[0]}"
    ids = tmp_path / "ids.txt"
    ids.write_text("\n".join(" ".join(map(str, p)) for p in prompts) + "\n")
    out = run(module + ["generate", str(folder), "--prompts-file", str(ids), "--max-tokens", "7", "--dtype", "float32"])
    assert [[int(t) for t in line.split()] for line in out.strip().splitlines()] == want
    sampled = run(module + ["generate", str(folder), "--prompts-file", str(ids), "--max-tokens", "7", "--temperature", "0.8", "--seed", "5"])
    assert sampled == run(module + ["generate", str(folder), "--prompts-file", str(ids), "--max-tokens", "7", "--temperature", "0.8", "--seed", "5"])
    assert all(len(line.split()) == 7 for line in sampled.strip().splitlines())
    # the trace runner: requests whole, in unequal batches, and with their last tokens one by one
    requests = {f"r{i}": random_tokens(n, pcfg["vocab"], 20 + i) for i, n in enumerate([40, 3, 21])}
    ref = {rid: plain.forward(pcfg, pw, t) for rid, t in requests.items()}
    for name, steps in (("whole", ts.whole(requests)), ("tail", ts.last_one_by_one(requests, 12)), ("batches", ts.batches(requests, 3))):
        out_dir = tmp_path / name
        stdout = run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", str(folder), "--dtype", "float32", "--out", str(out_dir),
                      "--max-tokens", str(ts.held_tokens(steps))], input="".join(json.dumps(s) + "\n" for s in steps))
        assert [l for l in stdout.splitlines() if l.startswith("done")] == [f"done {s['step']}" for s in steps]
        outputs = {s["step"]: np.fromfile(out_dir / f"{s['step']}.f32", dtype="<f4") for s in steps if any(e["want"] for e in s["entries"])}
        got = ts.collect(steps, outputs, pcfg["vocab"])
        for rid in requests:
            assert rel_l2(torch.from_numpy(got[rid]), ref[rid]) < 2e-5, (name, rid)
