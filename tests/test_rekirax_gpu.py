"""Rekirax through the engine on the GPU against the plain implementation (tests/plain_rekirax.py), in 32-bit
and in bfloat16: each mechanism alone, whole prompts against token-by-token decoding, portions down to two
tokens, mixed batches against each request alone, pages and state slots that are used again, keys at window,
chunk and page borders, the first tokens, long decoding, and greedy generation through the engine's own entry
point and scheduler."""
import numpy as np
import pytest

import plain_rekirax as pr
import rekirax_cases as rc
import replay_util as ru

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]


@pytest.fixture(scope="module")
def dirs(tmp_path_factory):
    from mini_llm_amd import write_random_model
    made = {}

    def get(name, seed=3):
        if name not in made:
            d = tmp_path_factory.mktemp("rekirax_" + name)
            write_random_model(dict(getattr(rc, name)), str(d), seed)
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
@pytest.mark.parametrize("name", ["ONLY_ATTENTION", "ONLY_ATTENTION_UNCAPPED", "ONLY_PAIR", "ONLY_PAIR_WIDE"])
def test_each_mechanism_alone(dirs, name, dtype):
    cfg, d = getattr(rc, name), dirs(name)
    reqs = rc.requests(cfg["vocab"], [1, 2, 3, 9, 37, 64, 65, 150], seed=5)
    for label, steps in (("whole", ru.trace_whole(reqs)), ("chunks", ru.trace_chunks(reqs, seed=1)),
                         ("decode", ru.trace_decode_tail(reqs, tail=20))):
        runner = _runner(d, dtype, n_pages=ru.peak_tokens(steps) // 4)
        rc.check_against_plain(d, reqs, steps, ru.run_in_process(runner, steps), dtype, cfg["vocab"], f"{name} {label}")
        assert runner.check() == "" and runner.info()["n_requests"] == 0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["LOOPED_A", "LOOPED_B", "SINGLE_PASS", "ODD"])
@pytest.mark.parametrize("family", ["whole", "decode", "chunks", "mixed"])
def test_schedule_families_match_plain(dirs, name, family, dtype):
    """Each request whole; most of it at once and the rest token by token; portions down to two tokens; up to
    four live requests in mixed batches. The pool holds just the peak of live tokens and there are four state
    slots for eight requests, so pages and slots are used again (and were filled with NaN before)."""
    cfg, d = getattr(rc, name), dirs(name)
    reqs = rc.requests(cfg["vocab"], [1, 2, 3, 4, 5, 29, 64, 71] + ([150] if name == "ODD" else []), seed=11)
    steps = _families(reqs, seed=2)[family]
    n_pages = ru.peak_tokens(steps) // 4
    runner = _runner(d, dtype, n_pages)
    rc.check_against_plain(d, reqs, steps, ru.run_in_process(runner, steps), dtype, cfg["vocab"], f"{name} {family}")
    info = runner.info()
    assert runner.check() == "" and info["free_pages"] == n_pages and info["n_requests"] == 0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("page", [8, 16, 64])
@pytest.mark.parametrize("family", ["whole", "decode", "chunks", "mixed"])
def test_on_the_kernels_shared_with_plain_attention(dirs, family, page, dtype):
    """Head sizes 64, 128 and 48 at pages of 8 to 64 tokens: prompt portions on the matrix-core tiles, single tokens on
    the split-key kernel, with shaped scores, chunks and gates handed on; prompts of up to 300 tokens (several key
    tiles, windows and chunks that end inside a tile), portions, and mixed batches whose single tokens ride along."""
    from mini_llm_amd.kernels import ops
    cfg, d = rc.SHARED_KERNELS, dirs("SHARED_KERNELS")
    reqs = rc.requests(cfg["vocab"], [1, 2, 17, 63, 64, 65, 130, 300], seed=71)
    steps = _families(reqs, seed=6)[family]
    ops.reset_seen()
    runner = _runner(d, dtype, n_pages=-(-ru.peak_tokens(steps) // page), page=page)
    rc.check_against_plain(d, reqs, steps, ru.run_in_process(runner, steps), dtype, cfg["vocab"], f"shared kernels page {page} {family}")
    if family == "whole":
        assert ops.seen("prefill_tile_launches" if dtype == "bfloat16" else "tiled_f32_launches") > 0
    assert runner.check() == "" and runner.info()["n_requests"] == 0


def test_shared_kernels_against_the_row_kernel(dirs):
    """The same steps with the shared kernels switched off (every row through the one-wavefront-per-row kernel):
    both round differently, no more."""
    from mini_llm_amd.kernels import ops
    cfg, d = rc.SHARED_KERNELS, dirs("SHARED_KERNELS")
    reqs = rc.requests(cfg["vocab"], [5, 100, 257], seed=72)
    steps, _ = ru.trace_mixed(reqs, seed=9, max_live=3, tail=20)
    got = []
    try:
        for on in (True, False):
            ops.set_scored_shared_kernels(on)
            ops.reset_seen()
            runner = _runner(d, "float32", n_pages=ru.peak_tokens(steps) // 16, page=16)
            got.append(ru.collect(steps, ru.run_in_process(runner, steps), cfg["vocab"]))
            assert (ops.seen("tiled_f32_launches") > 0) == on
    finally:
        ops.set_scored_shared_kernels(True)
    worst = max(rc.row_error(got[0][r][p], got[1][r][p].astype(np.float64)) for r in reqs for p in range(len(reqs[r])))
    print(f"shared kernels against the row kernel: {worst:.3e}")
    assert worst <= 2e-5


@pytest.mark.parametrize("page", [2, 4, 16])
def test_window_chunk_and_page_borders_with_peaked_scores(dirs, page):
    """Scores scaled so that single keys dominate, windows of 5 and 16 and chunks of 6 over pages of 2, 4 and 16
    tokens: a window or chunk that is one key off, or a key lost at a page's border, changes whole rows.
    Prompts, portions that start and end inside a chunk, and decoding."""
    cfg, d = rc.PEAKED, dirs("PEAKED")
    reqs = rc.requests(cfg["vocab"], [40, 23, 17], seed=21)
    for label, steps in (("whole", ru.trace_whole(reqs)), ("decode", ru.trace_decode_tail(reqs, tail=19)),
                         ("chunks", ru.trace_chunks(reqs, seed=3, sizes=(2, 5, 3, 16, 7, 2, 4)))):
        runner = _runner(d, "float32", n_pages=-(-ru.peak_tokens(steps) // page), page=page)
        rc.check_against_plain(d, reqs, steps, ru.run_in_process(runner, steps), "float32", cfg["vocab"], f"peaked page {page} {label}",
                               tol=rc.TOL_PEAKED)


@pytest.mark.parametrize("page", [4, 16])
def test_far_keys_among_hundreds_with_peaked_scores(dirs, page):
    """A window of 300 and chunks of 190 keys and scores that single keys dominate: a key far back that is lost (a
    page of the table, a tile's edge, a window that ends early) changes whole rows. 32-bit."""
    cfg, d = rc.PEAKED_FAR, dirs("PEAKED_FAR")
    reqs = rc.requests(cfg["vocab"], [400, 200], seed=23)
    for label, steps in (("whole", ru.trace_whole(reqs)), ("decode", ru.trace_decode_tail(reqs, tail=40)),
                         ("chunks", ru.trace_chunks(reqs, seed=4, sizes=(2, 70, 3, 129, 16)))):
        runner = _runner(d, "float32", n_pages=-(-ru.peak_tokens(steps) // page), page=page)
        rc.check_against_plain(d, reqs, steps, ru.run_in_process(runner, steps), "float32", cfg["vocab"], f"far keys page {page} {label}",
                               tol=rc.TOL_PEAKED)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_prompt_of_a_thousand_tokens(dirs, dtype):
    """One prompt of 1,100 tokens whole, in portions of hundreds and of two tokens, and with its last tokens one by
    one: many key tiles, many chunks of the scan, block tables of dozens of pages."""
    cfg, d = rc.SHARED_KERNELS, dirs("SHARED_KERNELS")
    reqs = rc.requests(cfg["vocab"], [1100], seed=81)
    for label, steps in (("whole", ru.trace_whole(reqs)), ("chunks", ru.trace_chunks(reqs, seed=8, sizes=(300, 2, 129, 64, 401))),
                         ("decode", ru.trace_decode_tail(reqs, tail=25))):
        runner = _runner(d, dtype, n_pages=ru.peak_tokens(steps) // 16, page=16)
        rc.check_against_plain(d, reqs, steps, ru.run_in_process(runner, steps), dtype, cfg["vocab"], f"long prompt {label}")


@pytest.mark.parametrize("what", ["window", "chunk"])
def test_peaked_scores_would_show_an_edge_one_key_off(dirs, what):
    """The tests above have teeth: the plain model with every window (or chunk) one key wider differs from the
    plain model by far more than the tolerance, in most rows."""
    import copy
    d = dirs("PEAKED")
    cfg, w = pr.read_model(d)
    off = copy.deepcopy(cfg)
    for l in off["layers"]:
        if l["type"] == "attention" and what == "window":
            l["mixer"]["mask"]["size"] += 1
        if l["type"] == "parallel" and what == "chunk":
            l["mixer"]["left"]["mask"]["size"] += 1
    toks = rc.requests(cfg["vocab"], [40], seed=21)["r0"]
    a, b = pr.forward(cfg, w, toks).numpy(), pr.forward(off, w, toks).numpy()
    errs = np.array([rc.row_error(b[p], a[p]) for p in range(8, 40)])
    assert (errs > 20 * rc.TOL_PEAKED).mean() > 0.8


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding_and_slots_used_again(dirs, dtype):
    """One state slot and a small pool: three requests one after the other, each a short prompt and then 150
    tokens one by one, every one of them compared; the slot and the pages are the same ones each time."""
    cfg, d = rc.LOOPED_A, dirs("LOOPED_A")
    reqs = rc.requests(cfg["vocab"], [153, 151, 152], seed=31)
    steps = ru.trace_decode_tail(reqs, tail=150)
    runner = _runner(d, dtype, n_pages=40, max_num_seqs=1)
    rc.check_against_plain(d, reqs, steps, ru.run_in_process(runner, steps), dtype, cfg["vocab"], "long decoding")
    assert runner.check() == "" and runner.info()["free_pages"] == 40


def test_batches_of_unequal_requests_equal_each_alone(dirs):
    """The logits of a position do not depend on what else is in the batch, beyond rounding: the mixed family's
    rows against the same requests run whole and alone, engine against engine, in bfloat16."""
    cfg, d = rc.LOOPED_B, dirs("LOOPED_B")
    reqs = rc.requests(cfg["vocab"], [3, 50, 18, 64, 7], seed=41)
    fam = _families(reqs, seed=4)
    got = {}
    for family in ("whole", "mixed"):
        runner = _runner(d, "bfloat16", n_pages=ru.peak_tokens(fam[family]) // 4)
        got[family] = ru.collect(fam[family], ru.run_in_process(runner, fam[family]), cfg["vocab"])
    worst = max(rc.row_error(got["mixed"][r][p], got["whole"][r][p].astype(np.float64)) for r in reqs for p in range(len(reqs[r])))
    print(f"mixed against alone, bfloat16: {worst:.3e}")
    assert worst <= 2e-2


def test_residual_stream_after_every_layer_run(dirs):
    """Layer by layer: models that stop after 1, 2, ... layers of LOOPED_A's list (the loop cut where the list ends)
    agree with the plain model's logits, so a fault is pinned to the first layer run that shows it."""
    import copy
    from mini_llm_amd import write_random_model
    import tempfile
    full = rc.LOOPED_A
    for n in range(1, len(full["layers"]) + 1):
        cfg = copy.deepcopy(full)
        cfg["layers"] = cfg["layers"][:n]
        if n <= cfg["loop"]["start"]:
            del cfg["loop"]
        else:
            cfg["loop"]["stop"] = min(cfg["loop"]["stop"], n)
        with tempfile.TemporaryDirectory() as d:
            write_random_model(cfg, d, 9)
            reqs = rc.requests(cfg["vocab"], [21], seed=n)
            steps = ru.trace_chunks(reqs, seed=n, sizes=(5, 2, 9))
            runner = _runner(d, "float32", n_pages=16)
            rc.check_against_plain(d, reqs, steps, ru.run_in_process(runner, steps), "float32", cfg["vocab"], f"first {n} layers")


@pytest.mark.parametrize("dtype", DTYPES)
def test_trace_run_program(dirs, tmp_path, dtype):
    """The mixed family through bin/trace_run as a user drives it (its default page size and four state slots)."""
    cfg, d = rc.LOOPED_A, dirs("LOOPED_A")
    reqs = rc.requests(cfg["vocab"], [2, 33, 64, 5, 70, 21], seed=51)
    steps, _ = ru.trace_mixed(reqs, seed=5, max_live=4, tail=5)
    out = ru.run_trace_run(d, dtype, steps, str(tmp_path / "out"), ru.peak_tokens(steps))
    rc.check_against_plain(d, reqs, steps, out, dtype, cfg["vocab"], "program mixed")


@pytest.mark.parametrize("dtype", DTYPES)
def test_greedy_generation_through_the_engine(dirs, dtype):
    """Engine.generate (scheduler, continuous batching, prompt portions of 7 tokens, two requests at a time for
    five prompts, pages of 4) against the plain model's greedy tokens."""
    from mini_llm_amd import Engine, EngineOptions, SamplingParams
    cfg_d, d = rc.LOOPED_A, dirs("LOOPED_A")
    cfg, w = pr.read_model(d)
    prompts = list(rc.requests(cfg_d["vocab"], [1, 6, 19, 30, 11], seed=61).values())
    engine = Engine.from_pretrained(d, dtype=dtype, options=EngineOptions(kv_block_size=4, total_kv_blocks=64, max_batch_num=2,
                                                                          max_tokens_per_step=16, prefill_chunk=7))
    outs = engine.generate(prompts, SamplingParams(max_new_tokens=9, ignore_eos=True))
    for p, o in zip(prompts, outs):
        assert len(o) == 9
        if dtype == "float32":
            assert o == pr.greedy_generate(cfg, w, p, 9)
        else:
            # bfloat16 may turn a near-tie: every token must be one the plain model chose or nearly chose
            ids = list(p)
            for t in o:
                row = pr.forward(cfg, w, ids)[-1]
                assert float(row[t]) >= float(row.max()) - 0.08 * float(row.std()), (o, t)
                ids.append(t)
