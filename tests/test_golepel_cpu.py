"""Golepel through the engine's host logic on the CPU (the product's model, cache, step function and generation loop
over the plain torch kernels of tests/ref_ops.py), against the plain implementation in tests/plain."""
import pytest
import torch

from trapetum_amd.config import ConfigError, GolepelConfig
from trapetum_amd.engine.generate import generate

from . import golepel_tiny as gt
from .cpu_engine import load_cpu_model
from .plain import golepel_plain as plain
from .tiny import random_tokens

TOL = 2e-5


@pytest.fixture(scope="module", params=["P", "Q"])
def m(request, tmp_path_factory):
    folder = gt.make_folder(tmp_path_factory.mktemp("g"), request.param)
    model, cfg = load_cpu_model(folder)
    pcfg, pw = plain.read_folder(folder)
    return model, cfg, pcfg, pw, TOL


@pytest.fixture(scope="module")
def sharp(tmp_path_factory):
    folder = gt.make_folder(tmp_path_factory.mktemp("g"), "S")
    model, cfg = load_cpu_model(folder)
    pcfg, pw = plain.read_folder(folder)
    # float32 rounding grows through softmaxes this sharp to some 1e-3 of the logits; a lost key costs tenths
    return model, cfg, pcfg, pw, 4e-3


def test_layout_and_cache(m):
    model, cfg, pcfg, _, _ = m
    names = set(model.tensor_layout())
    assert {"embed", "final.norm", "l0.norm1", "l0.canon1", "l0.mix.q", "l0.mix.dkv", "l0.mix.dkv.norm", "l0.mix.uk",
            "l0.mix.uv", "l0.mix.o", "l0.mlp.router", "l0.mlp.e0.gate"} <= names
    cache = model.new_cache(max_tokens=64, page_size=16)
    for i, layer in enumerate(pcfg["layers"]):
        mx = layer["mixer"]
        if "kv_from" in mx:                              # reads another run's rows, keeps none
            assert f"l{i}.mix.dkv" not in names and cache.site(i) is None
        else:                                            # one tensor per token: the rotated key part and the latent
            assert list(cache.site(i).spec.tensors) == [("latent", (1, mx["rot_dim"] + mx["kv_rank"]))]
        if layer["mlp"] is None:
            assert f"l{i}.norm2" not in names and f"l{i}.canon2" not in names
    taps = pcfg["canon"]["taps"]
    states = [s for e in model.entry_state_specs() for s in e.values()]
    if taps == 1:
        assert states == []
    else:
        assert all(s.shape == (taps - 1, pcfg["width"]) and s.dtype == "float32" for s in states)
        assert len(states) == sum(1 if l["mlp"] is None else 2 for l in pcfg["layers"])


def test_config_errors():
    d = gt.config_p()
    for path, value, match in [(("layers", 1, "mixer", "kv_from"), 3, "does not run before"),
                               (("layers", 1, "mixer", "kv_rank"), 16, "must be equal"),
                               (("layers", 3, "mixer", "kv_from"), 1, "no down-projection"),
                               (("norm", "groups"), 5, "divide"), (("layers", 0, "mlp", "router", "top"), 9, "top"),
                               (("layers", 0, "type"), "other", "latent_attention"), (("canon", "taps"), 0, "taps")]:
        bad = gt.config_p()
        at = bad
        for k in path[:-1]:
            at = at[k]
        at[path[-1]] = value
        with pytest.raises(ConfigError, match=match):
            GolepelConfig.from_dict(bad)
    del d["logit_scale"]
    with pytest.raises(ConfigError, match="logit_scale"):
        GolepelConfig.from_dict(d)


def test_whole_and_token_by_token(m):
    gt.whole_and_token_by_token(m, n=40)


def test_prompt_then_decode(m):
    gt.prompt_then_decode(m, n=50, tail=30)


def test_portions(m):
    gt.portions(m)


def test_unequal_batches_and_reuse(m):
    gt.unequal_batches_and_reuse(m)


def test_slot_after_a_longer_sequence(m):
    gt.slot_after_a_longer_sequence(m)


def test_sharp_scores_far_keys(sharp):
    gt.sharp_scores_far_keys(sharp, n=100)


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
