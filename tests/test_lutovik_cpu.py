"""Lutovik through the engine's host logic on the CPU (the product's model, cache, step function and generation loop
over the plain torch kernels of tests/ref_ops.py), against the plain implementation in tests/plain."""
import pytest
import torch

from trapetum_amd.config import ConfigError, LutovikConfig
from trapetum_amd.engine.generate import generate
from trapetum_amd.parts.rope import RotaryPosition

from . import lutovik_tiny as lt
from . import model_cases as mc
from .cpu_engine import load_cpu_model
from .plain import lutovik_plain as plain
from .tiny import random_tokens

TOL = 2e-5


@pytest.fixture(scope="module", params=["P", "Q"])
def m(request, tmp_path_factory):
    folder = lt.make_folder(tmp_path_factory.mktemp("l"), request.param)
    model, cfg = load_cpu_model(folder)
    pcfg, pw = plain.read_folder(folder)
    return model, cfg, pcfg, pw, TOL


@pytest.fixture(scope="module")
def sharp(tmp_path_factory):
    folder = lt.make_folder(tmp_path_factory.mktemp("l"), "S")
    model, cfg = load_cpu_model(folder)
    pcfg, pw = plain.read_folder(folder)
    # float32 rounding grows through softmaxes this sharp to some 1e-3 of the logits; a lost key costs tenths
    return model, cfg, pcfg, pw, 4e-3


def test_layout_cache_and_states(m):
    model, cfg, pcfg, _, _ = m
    names = set(model.tensor_layout())
    assert {"embed", "head", "final.norm"} <= names
    cache = model.new_cache(max_tokens=64, page_size=16)
    states = model.entry_state_specs()
    for i, layer in enumerate(pcfg["layers"]):
        mx = layer["mixer"]
        if layer["type"] == "attention":
            assert {f"l{i}.mix.q", f"l{i}.mix.o", f"l{i}.norm1", f"l{i}.norm1b"} <= names and states[i] == {}
            if "kv_from" in mx:                          # no projections of keys and values, no cache of its own
                assert f"l{i}.mix.k" not in names and f"l{i}.mix.v" not in names and cache.site(i) is None
                continue
            att = mx
        else:
            att, r = mx["left"], mx["right"]
            assert {f"l{i}.mix.left.g", f"l{i}.mix.left.out", f"l{i}.mix.right.out", f"l{i}.mix.right.conv.b",
                    f"l{i}.mix.right.A_log"} <= names
            want = {"mixer.right.ssm": (r["heads"], r["state"], r["vdim"])}
            if r["conv"] > 1:
                want["mixer.right.conv"] = (r["conv"] - 1, r["heads"] * r["vdim"] + 2 * r["groups"] * r["state"])
            assert {k: v.shape for k, v in states[i].items()} == want
            assert all(v.dtype == "float32" for v in states[i].values())
        row = max(att["dim"], att["vdim"])               # keys and values share rows of the larger size
        assert list(cache.site(i).spec.tensors) == [("k", (att["kv_heads"], row)), ("v", (att["kv_heads"], row))]
        if layer["mlp"] is None:
            assert f"l{i}.norm2" not in names and f"l{i}.norm2b" not in names
        elif layer["mlp"]["kind"] == "moe":
            assert (f"l{i}.mlp.shared.gate" in names) == ("shared" in layer["mlp"])


def test_config_errors():
    for path, value, match in [(("layers", 2, "mixer", "kv_from"), 3, "does not run before"),
                               (("layers", 2, "mixer", "kv_from"), 1, "no attention with keys"),
                               (("layers", 5, "mixer", "kv_from"), 0, "must be equal"),
                               (("layers", 0, "mixer", "kv_heads"), 3, "no multiple"),
                               (("layers", 0, "mixer", "rot", "dims"), 18, "exceeds dim"),
                               (("layers", 0, "mixer", "rot", "scaling", "high"), 0.5, "high above low"),
                               (("layers", 1, "mixer", "right", "groups"), 3, "groups"),
                               (("layers", 1, "mixer", "right", "norm_groups"), 5, "norm_groups"),
                               (("layers", 1, "mixer", "left", "kv_from"), 0, "of its own"),
                               (("layers", 1, "mlp", "router", "top"), 9, "top"),
                               (("layers", 0, "type"), "other", "attention and parallel")]:
        bad = lt.config_p()
        at = bad
        for k in path[:-1]:
            at = at[k]
        at[path[-1]] = value
        with pytest.raises(ConfigError, match=match):
            LutovikConfig.from_dict(bad)
    d = lt.config_p()
    del d["embedding"]
    with pytest.raises(ConfigError, match="embedding"):
        LutovikConfig.from_dict(d)


@pytest.mark.parametrize("base,dims,scaling", [(500.0, 8, (8.0, 1.0, 3.0, 64)), (10000.0, 32, (6.0, 1.0, 5.0, 256)),
                                               (3000.0, 12, (2.5, 2.0, 9.0, 100)), (77.0, 24, None)])
def test_scaled_frequencies(base, dims, scaling):
    sc = None if scaling is None else dict(zip(("factor", "low", "high", "original"), scaling))
    want = plain.frequencies(base, dims, sc)
    got = RotaryPosition(dims, base, scaling=sc).inv_freq("cpu").double()
    assert float(((got - want) / want).abs().max()) < 5e-7
    if scaling is not None:                              # the case has frequencies of all three kinds
        plainf = plain.frequencies(base, dims, None)
        ratio = want / plainf
        assert bool((ratio == 1).any()) and bool((ratio - 1 / scaling[0]).abs().min() < 1e-12) and \
            bool(((ratio < 1 - 1e-9) & (ratio > 1 / scaling[0] + 1e-9)).any())


def test_whole_and_token_by_token(m):
    mc.whole_and_token_by_token(m, n=40)


def test_prompt_then_decode(m):
    mc.prompt_then_decode(m, n=50, tail=30)


def test_portions(m):
    mc.portions(m)


def test_unequal_batches_and_reuse(m):
    mc.unequal_batches_and_reuse(m)


def test_slot_after_a_longer_sequence(m):
    mc.slot_after_a_longer_sequence(m)


def test_sharp_scores_far_keys(sharp):
    mc.sharp_scores_far_keys(sharp, n=100)


def test_a_far_key_decides(sharp):
    """The sharp model's logits at the end of a long sequence change when one early token changes, by as much as the
    plain implementation says: the early key is seen, through the cache, from a decoded token."""
    model, cfg, pcfg, pw, _ = sharp
    a = random_tokens(120, cfg.vocab_size, 61)
    found = False
    for at in (1, 2, 3, 5, 8):
        b = list(a)
        b[at] = (a[at] + 1) % cfg.vocab_size
        ra, rb = plain.forward(pcfg, pw, a)[-1], plain.forward(pcfg, pw, b)[-1]
        if float((ra - rb).norm() / ra.norm()) < 1e-3:
            continue
        found = True
        cache = model.new_cache(max_tokens=256, page_size=16)
        outs = []
        for toks in (a, b):
            s = cache.acquire()
            model.step(cache, [s], toks[:100], counts=[100], want=[])
            outs.append(torch.cat([model.step(cache, [s], [t]) for t in toks[100:]])[-1].double())
            cache.release(s)
        assert float(((outs[0] - outs[1]) - (ra - rb)).norm() / (ra - rb).norm()) < 1e-3, at
    assert found


def test_greedy_generation_through_the_loop(m):
    model, cfg, pcfg, pw, _ = m
    prompts = [random_tokens(n, cfg.vocab_size, 70 + n) for n in (7, 1, 19, 4)]
    want = [plain.greedy_generate(pcfg, pw, p, 6) for p in prompts]
    cache = model.new_cache(max_tokens=64 * 2, page_size=64)             # room for two sequences at a time: slots are used again
    assert generate(model, cache, prompts, max_tokens=6, stop_ids=()) == want
    assert cache.live_slots() == [] and cache.tokens_held() == 0


@pytest.mark.parametrize("case", range(6))
def test_random_configuration(case, tmp_path):
    """A configuration drawn at random: a prompt whole, then in two portions and single tokens."""
    import random

    from trapetum_amd.weights import write_model_folder

    from .lutovik_random import draw
    rng = random.Random(500 + case)
    cfg = draw(rng)
    folder = str(tmp_path)
    write_model_folder(LutovikConfig.from_dict(cfg), folder, seed=case, sigma=0.1, sigma_norm=0.2)
    model, c = load_cpu_model(folder)
    pcfg, pw = plain.read_folder(folder)
    assert pcfg == cfg
    toks = random_tokens(37, c.vocab_size, case)
    ref = plain.forward(pcfg, pw, toks)
    cache = model.new_cache(max_tokens=128, page_size=16)
    s = cache.acquire()
    got = [model.step(cache, [s], toks[:20], counts=[20], want=list(range(20))),
           model.step(cache, [s], toks[20:31], counts=[11], want=list(range(11)))]
    got += [model.step(cache, [s], [t]) for t in toks[31:]]
    mc.rows_close(torch.cat(got), ref, 5e-5, cfg)
