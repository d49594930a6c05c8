"""Kugulorn through the engine on the GPU against the plain implementation (tests/plain_kugulorn.py), in
32-bit and in bfloat16: each mechanism alone, whole prompts against token-by-token decoding, portions down
to two tokens, mixed batches against each request alone, pages and state slots that are used again, keys at
window and page borders, the first tokens, long decoding, and greedy generation through the engine's own
entry point and scheduler."""
import numpy as np
import pytest

import kugulorn_cases as kc
import plain_kugulorn as pk
import replay_util as ru

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]


@pytest.fixture(scope="module")
def dirs(tmp_path_factory):
    from mini_llm_amd import write_random_model
    made = {}

    def get(name, seed=3):
        if name not in made:
            d = tmp_path_factory.mktemp("kugulorn_" + name)
            write_random_model(dict(getattr(kc, name)), str(d), seed)
            made[name] = str(d)
        return made[name]
    return get


def _runner(model_dir, dtype, n_pages, page=4, max_num_seqs=4):
    from mini_llm_amd import Runner
    r = Runner(model_dir=model_dir, dtype=dtype, page_size=page, n_pages=n_pages, max_num_seqs=max_num_seqs)
    r.poison_cache()               # a stale or unwritten page or slot that is read shows up as NaN
    return r


def _families(reqs, seed):
    mixed, _ = ru.trace_mixed(reqs, seed=seed, max_live=4, tail=6)
    return {"whole": ru.trace_whole(reqs), "decode": ru.trace_decode_tail(reqs, tail=11),
            "chunks": ru.trace_chunks(reqs, seed=seed), "mixed": mixed}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["ONLY_MAMBA", "ONLY_MAMBA_WIDE_STATE", "ONLY_LATENT", "ONLY_LATENT_MLP"])
def test_each_mechanism_alone(dirs, name, dtype):
    cfg, d = getattr(kc, name), dirs(name)
    # (portions of more than 64 tokens: the scan cuts them into chunks that run side by side)
    reqs = kc.requests(cfg["vocab"], [1, 2, 3, 9, 37, 64, 65, 200], seed=5)
    for label, steps in (("whole", ru.trace_whole(reqs)), ("chunks", ru.trace_chunks(reqs, seed=1)),
                         ("long chunks", ru.trace_chunks(reqs, seed=1, sizes=(70, 3, 129)))):
        runner = _runner(d, dtype, n_pages=ru.peak_tokens(steps) // 4)
        kc.check_against_plain(d, reqs, steps, ru.run_in_process(runner, steps), dtype, cfg["vocab"], f"{name} {label}")
        assert runner.check() == "" and runner.info()["n_requests"] == 0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["MIXED_A", "MIXED_B", "ODD"])
@pytest.mark.parametrize("family", ["whole", "decode", "chunks", "mixed"])
def test_schedule_families_match_plain(dirs, name, family, dtype):
    """Each request whole; most of it at once and the rest token by token; portions down to two tokens; up to
    four live requests in mixed batches. The pool holds just the peak of live tokens and there are four state
    slots for seven requests, so pages and slots are used again (and were filled with NaN before)."""
    cfg, d = getattr(kc, name), dirs(name)
    reqs = kc.requests(cfg["vocab"], [1, 2, 3, 4, 5, 29, 64, 71] + ([150] if name == "ODD" else []), seed=11)
    steps = _families(reqs, seed=2)[family]
    n_pages = ru.peak_tokens(steps) // 4
    runner = _runner(d, dtype, n_pages)
    kc.check_against_plain(d, reqs, steps, ru.run_in_process(runner, steps), dtype, cfg["vocab"], f"{name} {family}")
    info = runner.info()
    assert runner.check() == "" and info["free_pages"] == n_pages and info["n_requests"] == 0


@pytest.mark.parametrize("page", [8, 16, 64])
@pytest.mark.parametrize("family", ["whole", "decode", "chunks", "mixed"])
def test_prompt_portions_on_the_matrix_cores(dirs, family, page):
    """bfloat16 at sizes and page sizes that the matrix-core kernel takes: prompts of up to 300 tokens (several
    key tiles, windows that end inside a tile), portions, and mixed batches whose single tokens ride along."""
    from mini_llm_amd.kernels import ops
    cfg, d = kc.TILED, dirs("TILED")
    reqs = kc.requests(cfg["vocab"], [1, 2, 17, 63, 64, 65, 130, 300], seed=71)
    steps = _families(reqs, seed=6)[family]
    ops.reset_seen()
    runner = _runner(d, "bfloat16", n_pages=-(-ru.peak_tokens(steps) // page), page=page)
    kc.check_against_plain(d, reqs, steps, ru.run_in_process(runner, steps), "bfloat16", cfg["vocab"], f"tiled page {page} {family}")
    assert ops.seen("latent_tile_launches") > 0
    assert runner.check() == "" and runner.info()["n_requests"] == 0


@pytest.mark.parametrize("family", ["whole", "mixed"])
def test_widest_rows_on_the_matrix_cores(dirs, family):
    from mini_llm_amd.kernels import ops
    cfg, d = kc.WIDE, dirs("WIDE")
    reqs = kc.requests(cfg["vocab"], [3, 70, 129, 260], seed=73)
    steps = _families(reqs, seed=7)[family]
    ops.reset_seen()
    runner = _runner(d, "bfloat16", n_pages=ru.peak_tokens(steps) // 16, page=16)
    kc.check_against_plain(d, reqs, steps, ru.run_in_process(runner, steps), "bfloat16", cfg["vocab"], f"wide {family}")
    assert ops.seen("latent_tile_launches") > 0 and ops.seen("latent_token_launches") == 0


def test_matrix_core_kernel_against_the_per_token_kernel(dirs):
    """The same whole prompts with the matrix-core kernel switched off: both kernels round differently, no more."""
    from mini_llm_amd.kernels import ops
    cfg, d = kc.TILED, dirs("TILED")
    reqs = kc.requests(cfg["vocab"], [5, 100, 257], seed=72)
    steps = ru.trace_whole(reqs)
    got = []
    try:
        for on in (True, False):
            ops.set_latent_tiles(on)
            ops.reset_seen()
            runner = _runner(d, "bfloat16", n_pages=ru.peak_tokens(steps) // 16, page=16)
            got.append(ru.collect(steps, ru.run_in_process(runner, steps), cfg["vocab"]))
            assert (ops.seen("latent_tile_launches") > 0) == on
    finally:
        ops.set_latent_tiles(True)
    worst = max(kc.row_error(got[0][r][p], got[1][r][p].astype(np.float64)) for r in reqs for p in range(len(reqs[r])))
    print(f"matrix-core kernel against the per-token kernel: {worst:.3e}")
    assert worst <= 2e-2


@pytest.mark.parametrize("page", [2, 4, 16])
def test_window_and_page_borders_with_peaked_scores(dirs, page):
    """Scores scaled so that single keys dominate, windows of 5, 6 and 16 over pages of 2, 4 and 16 tokens: a
    window that is one key off or a key lost at a page's border changes whole rows. Prompts and decoding."""
    cfg, d = kc.PEAKED, dirs("PEAKED")
    reqs = kc.requests(cfg["vocab"], [40, 23, 17], seed=21)
    for label, steps in (("whole", ru.trace_whole(reqs)), ("decode", ru.trace_decode_tail(reqs, tail=19)),
                         ("chunks", ru.trace_chunks(reqs, seed=3, sizes=(2, 5, 3, 16, 7, 2, 4)))):
        runner = _runner(d, "float32", n_pages=-(-ru.peak_tokens(steps) // page), page=page)
        kc.check_against_plain(d, reqs, steps, ru.run_in_process(runner, steps), "float32", cfg["vocab"], f"peaked page {page} {label}",
                               tol=kc.TOL_PEAKED)


@pytest.mark.parametrize("page", [4, 16])
def test_far_keys_among_hundreds_with_peaked_scores(dirs, page):
    """Windows of 300 and 190 keys and scores that single keys dominate: a key far back that is lost (a page of the
    table, a tile's edge, a window that ends early) changes whole rows. Prompts, portions and decoding, 32-bit."""
    cfg, d = kc.PEAKED_FAR, dirs("PEAKED_FAR")
    reqs = kc.requests(cfg["vocab"], [330, 200], seed=23)
    for label, steps in (("whole", ru.trace_whole(reqs)), ("decode", ru.trace_decode_tail(reqs, tail=40)),
                         ("chunks", ru.trace_chunks(reqs, seed=4, sizes=(2, 70, 3, 129, 16)))):
        runner = _runner(d, "float32", n_pages=-(-ru.peak_tokens(steps) // page), page=page)
        kc.check_against_plain(d, reqs, steps, ru.run_in_process(runner, steps), "float32", cfg["vocab"], f"far keys page {page} {label}",
                               tol=kc.TOL_PEAKED)


def test_peaked_scores_would_show_a_window_one_key_off(dirs):
    """The test above has teeth: the plain model with every window one key wider differs from the plain model
    by far more than the tolerance, in most rows."""
    import copy
    d = dirs("PEAKED")
    cfg, w = pk.read_model(d)
    off = copy.deepcopy(cfg)
    for l in off["layers"]:
        l["mixer"]["mask"]["size"] += 1
    toks = kc.requests(cfg["vocab"], [40], seed=21)["r0"]
    a, b = pk.forward(cfg, w, toks).numpy(), pk.forward(off, w, toks).numpy()
    errs = np.array([kc.row_error(b[p], a[p]) for p in range(8, 40)])
    assert (errs > 20 * kc.TOL_PEAKED).mean() > 0.8


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding_and_slots_used_again(dirs, dtype):
    """One state slot and a small pool: three requests one after the other, each a short prompt and then 150
    tokens one by one, every one of them compared; the slot and the pages are the same ones each time."""
    cfg, d = kc.MIXED_A, dirs("MIXED_A")
    reqs = kc.requests(cfg["vocab"], [153, 151, 152], seed=31)
    steps = ru.trace_decode_tail(reqs, tail=150)
    runner = _runner(d, dtype, n_pages=40, max_num_seqs=1)
    kc.check_against_plain(d, reqs, steps, ru.run_in_process(runner, steps), dtype, cfg["vocab"], "long decoding")
    assert runner.check() == "" and runner.info()["free_pages"] == 40


def test_batches_of_unequal_requests_equal_each_alone(dirs):
    """The logits of a position do not depend on what else is in the batch, beyond rounding: the mixed family's
    rows against the same requests run whole and alone, engine against engine, in bfloat16."""
    cfg, d = kc.MIXED_B, dirs("MIXED_B")
    reqs = kc.requests(cfg["vocab"], [3, 50, 18, 64, 7], seed=41)
    fam = _families(reqs, seed=4)
    got = {}
    for family in ("whole", "mixed"):
        runner = _runner(d, "bfloat16", n_pages=ru.peak_tokens(fam[family]) // 4)
        got[family] = ru.collect(fam[family], ru.run_in_process(runner, fam[family]), cfg["vocab"])
    worst = max(kc.row_error(got["mixed"][r][p], got["whole"][r][p].astype(np.float64)) for r in reqs for p in range(len(reqs[r])))
    print(f"mixed against alone, bfloat16: {worst:.3e}")
    assert worst <= 2e-2


@pytest.mark.parametrize("dtype", DTYPES)
def test_trace_run_program(dirs, tmp_path, dtype):
    """The mixed family through bin/trace_run as a user drives it (its default page size and four state slots)."""
    cfg, d = kc.MIXED_A, dirs("MIXED_A")
    reqs = kc.requests(cfg["vocab"], [2, 33, 64, 5, 70, 21], seed=51)
    steps, _ = ru.trace_mixed(reqs, seed=5, max_live=4, tail=5)
    out = ru.run_trace_run(d, dtype, steps, str(tmp_path / "out"), ru.peak_tokens(steps))
    kc.check_against_plain(d, reqs, steps, out, dtype, cfg["vocab"], "program mixed")


@pytest.mark.parametrize("dtype", DTYPES)
def test_greedy_generation_through_the_engine(dirs, dtype):
    """Engine.generate (scheduler, continuous batching, prompt portions of 7 tokens, two requests at a time for
    five prompts, pages of 4) against the plain model's greedy tokens."""
    import torch
    from mini_llm_amd import Engine, EngineOptions, SamplingParams
    cfg_d, d = kc.MIXED_A, dirs("MIXED_A")
    cfg, w = pk.read_model(d)
    prompts = list(kc.requests(cfg_d["vocab"], [1, 6, 19, 30, 11], seed=61).values())
    engine = Engine.from_pretrained(d, dtype=dtype, options=EngineOptions(kv_block_size=4, total_kv_blocks=64, max_batch_num=2,
                                                                          max_tokens_per_step=16, prefill_chunk=7))
    outs = engine.generate(prompts, SamplingParams(max_new_tokens=9, ignore_eos=True))
    for p, o in zip(prompts, outs):
        assert len(o) == 9
        if dtype == "float32":
            assert o == pk.greedy_generate(cfg, w, p, 9)
        else:
            # bfloat16 may turn a near-tie: every token must be one the plain model chose or nearly chose
            ids = list(p)
            for t in o:
                row = pk.forward(cfg, w, ids)[-1]
                assert float(row[t]) >= float(row.max()) - 0.08 * float(row.std()), (o, t)
                ids.append(t)
