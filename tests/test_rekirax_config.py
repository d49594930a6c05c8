"""Rekirax without a GPU: what its configuration asks of a checkpoint, what it refuses, and the plain
implementation's own consistency (the recurrence carried over a cut, masks at their edges, the order of runs)."""
import copy

import pytest
import torch

import plain_rekirax as pr
import rekirax_cases as rc
from mini_llm_amd import check_model_dir, describe_config, registered_architectures, write_random_model
from mini_llm_amd.config import ConfigError
from mini_llm_amd.weights import WeightsError


def test_registered_and_tensors_follow_the_layer_list():
    assert "Rekirax" in registered_architectures()
    d = describe_config(rc.LOOPED_A)
    assert d["architecture"] == "Rekirax"
    shapes = {t["name"]: t["shape"] for t in d["tensors"]}
    assert shapes["embed"] == [257, 64] and "head" not in shapes and shapes["final.norm"] == [64] and shapes["embed.norm"] == [64]
    assert shapes["loop.in"] == [64, 128] and shapes["loop.step"] == [2, 64]
    assert shapes["l0.mix.left.q"] == [64, 64] and shapes["l0.mix.left.k"] == [32, 64] and shapes["l0.mix.left.q.norm"] == [64]
    assert shapes["l2.mix.left.v"] == [3 * 24, 64] and shapes["l2.mix.left.g"] == [6 * 24, 64] and shapes["l2.mix.left.o"] == [64, 6 * 24]
    assert shapes["l2.mix.right.f"] == [64, 64] and shapes["l2.mix.right.norm"] == [8] and shapes["l2.mix.right.lower"] == [64]
    assert shapes["l1.mix.q"] == [64, 64] and shapes["l1.mix.k"] == [32, 64] and "l1.mix.v" not in shapes
    assert shapes["l1.mix.q.norm"] == [16] and shapes["l3.mix.r1"] == [2] and shapes["l1.canon1"] == [64, 3]
    assert "l2.norm2" not in shapes and shapes["l3.mlp.gate.b"] == [96] and shapes["l3.mlp.down"] == [64, 96]
    roles = {t["name"]: t["role"] for t in d["tensors"]}
    assert roles["l0.mix.right.lower"] == "vector" and roles["l0.mix.right.f"] == "matrix" and roles["loop.step"] == "vector"
    # neither a loop nor a convolution: their tensors are not asked for
    bare = {t["name"] for t in describe_config(rc.ONLY_PAIR_WIDE)["tensors"]}
    assert "loop.in" not in bare and "l0.canon1" not in bare


@pytest.mark.parametrize("change, message", [
    (lambda c: c["layers"][1].__setitem__("type", "lstm"), "unknown layer type"),
    (lambda c: c["layers"][1]["mixer"].__setitem__("kv_heads", 3), "multiple of kv_heads"),
    (lambda c: c["layers"][1]["mixer"].__setitem__("vdim", 8), "vdim must equal dim"),
    (lambda c: c["layers"][0]["mixer"]["left"]["rot"].__setitem__("dims", 7), "even"),
    (lambda c: c["layers"][0]["mixer"]["left"]["rot"].__setitem__("dims", 18), "at most dim"),
    (lambda c: c["layers"][0]["mlp"].__setitem__("kind", "routed"), "dense"),
    (lambda c: c["layers"][0]["mixer"].pop("right"), "right"),
    (lambda c: c["layers"][1]["mixer"].pop("mask"), "mask"),
    (lambda c: c["loop"].__setitem__("stop", 6), "start < stop"),
    (lambda c: c["loop"].__setitem__("start", 4), "start < stop"),
    (lambda c: c["canon"].__setitem__("taps", 17), "16 taps"),
    (lambda c: c.pop("norm"), "norm"),
])
def test_refusals(change, message):
    cfg = copy.deepcopy(rc.LOOPED_A)
    change(cfg)
    with pytest.raises(ConfigError, match=message):
        describe_config(cfg)


def test_written_folder_checks_and_a_missing_tensor_is_named(tmp_path):
    d = write_random_model(dict(rc.LOOPED_B), str(tmp_path / "m"), 1)
    arch, n_tensors, _ = check_model_dir(d)
    assert arch == "Rekirax" and n_tensors == len(describe_config(rc.LOOPED_B)["tensors"])
    from safetensors.torch import load_file, save_file
    t = load_file(str(tmp_path / "m" / "model.safetensors"))
    # the norm weights are written as they are stored: around zero
    assert float(t["l0.norm1"].abs().max()) < 1.0 and abs(float(t["l0.mix.q.norm"].mean()) - 1.0) < 0.2
    del t["l1.mix.right.lower"]
    save_file(t, str(tmp_path / "m" / "model.safetensors"))
    with pytest.raises(WeightsError, match="l1.mix.right.lower"):
        check_model_dir(d)


def test_order_of_layer_runs():
    assert pr.layer_runs(rc.LOOPED_A) == [(0, None), (1, 0), (2, None), (3, None), (1, 1), (2, None), (3, None), (4, None)]
    assert pr.layer_runs(rc.LOOPED_B) == [(0, 0), (1, None), (0, 1), (1, None), (0, 2), (1, None)]
    assert pr.layer_runs(rc.ONLY_PAIR) == [(0, None)]


def test_masks_at_their_edges():
    w = pr.visible(20, "window", 5)
    assert bool(w[10, 6]) and not bool(w[10, 5]) and bool(w[10, 10]) and not bool(w[10, 11]) and bool(w[2, 0])
    c = pr.visible(20, "chunk", 6)
    assert bool(c[11, 6]) and not bool(c[11, 5]) and not bool(c[12, 11]) and bool(c[12, 12]) and not bool(c[5, 6])


def test_plain_recurrence_carried_over_a_cut(tmp_path):
    """The plain HGRN2 run over a sequence equals the same run cut in two with the state handed on; and the gate's
    lower bound is honoured: with the gate's bias far below zero the state forgets at exactly the lower bound."""
    d = write_random_model(dict(rc.ONLY_PAIR), str(tmp_path / "m"), 2)
    cfg, w = pr.read_model(d)
    m, P, eps = cfg["layers"][0]["mixer"]["right"], "l0.mix.right.", cfg["norm"]["eps"]
    g = torch.Generator().manual_seed(0)
    h = torch.randn(13, cfg["width"], generator=g, dtype=torch.float64)
    whole = pr.hgrn2(h, w, P, m, eps)
    # the first 6 tokens, then the rest from the state they leave: worked out by the function's own recurrence
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    S = torch.zeros(H, dk, dv, dtype=torch.float64)
    low = w[P + "lower"]
    f = (low + (1 - low) * torch.sigmoid(h @ w[P + "f"].T + w[P + "f.b"])).reshape(13, H, dk)
    v = (h @ w[P + "v"].T).reshape(13, H, dv)
    for t in range(6):
        S = f[t][:, :, None] * S + (1 - f[t])[:, :, None] * v[t][:, None, :]
    rest = pr.hgrn2(h[6:], w, P, m, eps, state=S)
    assert torch.allclose(rest, whole[6:], atol=1e-12)
    assert float(f.min()) >= float(low.min()) - 1e-12 and float(f.max()) <= 1.0


def test_plain_prompt_equals_token_by_token_through_the_convolution(tmp_path):
    """The input convolution sees at most taps - 1 earlier rows: logits of a prefix do not depend on what follows."""
    d = write_random_model(dict(rc.SINGLE_PASS), str(tmp_path / "m"), 4)
    cfg, w = pr.read_model(d)
    toks = rc.requests(cfg["vocab"], [17], seed=3)["r0"]
    full = pr.forward(cfg, w, toks)
    for n in (1, 5, 12):
        assert torch.allclose(pr.forward(cfg, w, toks[:n]), full[:n], atol=1e-10)


@pytest.mark.parametrize("size", ["gpt2-small", "gpt2-medium", "gpt2-xl"])
def test_the_benchmark_configuration_is_a_model(size):
    """bench.py --design rekirax: its configuration at every size is one the architecture takes, with as many layer
    runs as the GPT-2 configuration of that size has layers."""
    import os
    import sys
    sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    import bench
    cfg = bench.rekirax_config(0, size)
    d = describe_config(cfg)
    assert d["architecture"] == "Rekirax"
    assert len(pr.layer_runs(cfg)) == bench.SIZES[size][0] == cfg["n_layer"]
    shapes = {t["name"]: t["shape"] for t in d["tensors"]}
    assert shapes["embed"][1] == bench.SIZES[size][1] and "loop.in" in shapes
