"""Sunulorn through the engine on the GPU against the plain implementation (tests/plain_sunulorn.py), in 32-bit
and in bfloat16: each mechanism alone, whole prompts against token-by-token decoding, portions down to two
tokens, mixed batches against each request alone, pages and state slots that are used again, keys at window
and page borders, kept first tokens and far keys, the first tokens, long decoding, and greedy generation through
the engine's own entry point and scheduler."""
import copy

import numpy as np
import pytest

import plain_sunulorn as ps
import replay_util as ru
import sunulorn_cases as sc

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]


@pytest.fixture(scope="module")
def dirs(tmp_path_factory):
    from mini_llm_amd import write_random_model
    made = {}

    def get(name, seed=3):
        if name not in made:
            d = tmp_path_factory.mktemp("sunulorn_" + name)
            write_random_model(dict(getattr(sc, name)), str(d), seed)
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


SINGLE = ["ONLY_CONV", "ONLY_CONV_BARE", "ONLY_CONV_ONE_TAP", "ONLY_CONV_LONG", "ONLY_CONV_MANY_TAPS", "ONLY_WINDOW", "ONLY_WINDOW_NO_KEEP",
          "ONLY_WINDOW_OPEN", "ONLY_WINDOW_KEEP_WIDE", "ONLY_SINK", "ONLY_SINK_ONE_HEAD", "ONLY_SINK_MANY", "SHARED_KV",
          "ONLY_DENSE", "ONLY_EXPERTS", "ONLY_EXPERTS_ALL", "ONE_EXPERT", "TOP_ONE", "SINK_SOFT"]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", SINGLE)
def test_each_mechanism_alone(dirs, name, dtype):
    cfg, d = getattr(sc, name), dirs(name)
    reqs = sc.requests(cfg["vocab"], [1, 2, 3, 9, 37, 64, 65, 150], seed=5)
    for label, steps in (("whole", ru.trace_whole(reqs)), ("chunks", ru.trace_chunks(reqs, seed=1)),
                         ("decode", ru.trace_decode_tail(reqs, tail=20))):
        runner = _runner(d, dtype, n_pages=ru.peak_tokens(steps) // 4)
        sc.check_against_plain(d, reqs, steps, ru.run_in_process(runner, steps), dtype, cfg["vocab"], f"{name} {label}")
        assert runner.check() == "" and runner.info()["n_requests"] == 0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["MIXED_A", "MIXED_B", "ODD", "UNUSUAL"])
@pytest.mark.parametrize("family", ["whole", "decode", "chunks", "mixed"])
def test_schedule_families_match_plain(dirs, name, family, dtype):
    """Each request whole; most of it at once and the rest token by token; portions down to two tokens; up to
    four live requests in mixed batches. The pool holds just the peak of live tokens and there are four state
    slots for eight requests, so pages and slots are used again (and were filled with NaN before)."""
    cfg, d = getattr(sc, name), dirs(name)
    reqs = sc.requests(cfg["vocab"], [1, 2, 3, 4, 5, 29, 64, 71] + ([150] if name in ("ODD", "UNUSUAL") else []), seed=11)
    steps = _families(reqs, seed=2)[family]
    n_pages = ru.peak_tokens(steps) // 4
    runner = _runner(d, dtype, n_pages)
    sc.check_against_plain(d, reqs, steps, ru.run_in_process(runner, steps), dtype, cfg["vocab"], f"{name} {family}")
    info = runner.info()
    assert runner.check() == "" and info["free_pages"] == n_pages and info["n_requests"] == 0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("page", [8, 16, 64])
@pytest.mark.parametrize("family", ["whole", "decode", "chunks", "mixed"])
def test_sizes_of_a_larger_models_layers(dirs, family, page, dtype):
    """Heads of 32, 64 and 128 at pages of 8 to 64 tokens; prompts of up to 300 tokens (several key tiles, windows that
    end inside a tile, kept tokens in a tile of their own), portions, and mixed batches whose single tokens ride along."""
    cfg, d = sc.LARGER, dirs("LARGER")
    reqs = sc.requests(cfg["vocab"], [1, 2, 17, 63, 64, 65, 130, 300], seed=71)
    steps = _families(reqs, seed=6)[family]
    runner = _runner(d, dtype, n_pages=-(-ru.peak_tokens(steps) // page), page=page)
    sc.check_against_plain(d, reqs, steps, ru.run_in_process(runner, steps), dtype, cfg["vocab"], f"larger page {page} {family}")
    assert runner.check() == "" and runner.info()["n_requests"] == 0


@pytest.mark.parametrize("page", [2, 4, 16])
def test_window_and_page_borders_with_peaked_scores(dirs, page):
    """Scores scaled so that single keys dominate, windows of 5 and 16 that keep 2 and 7 first tokens, over pages of
    2, 4 and 16 tokens: a window or a kept range that is one key off, or a key lost at a page's border, changes whole
    rows. Prompts, portions that start and end inside a window, and decoding."""
    cfg, d = sc.PEAKED, dirs("PEAKED")
    reqs = sc.requests(cfg["vocab"], [40, 23, 17], seed=21)
    for label, steps in (("whole", ru.trace_whole(reqs)), ("decode", ru.trace_decode_tail(reqs, tail=19)),
                         ("chunks", ru.trace_chunks(reqs, seed=3, sizes=(2, 5, 3, 16, 7, 2, 4)))):
        runner = _runner(d, "float32", n_pages=-(-ru.peak_tokens(steps) // page), page=page)
        sc.check_against_plain(d, reqs, steps, ru.run_in_process(runner, steps), "float32", cfg["vocab"], f"peaked page {page} {label}",
                               tol=sc.TOL_PEAKED)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["PEAKED_TILES_32", "PEAKED_TILES_64", "PEAKED_TILES_128", "SINK_TILES_64", "CONV_TILES_128"])
def test_masks_at_the_tiled_kernels_head_sizes(dirs, name, dtype):
    """Windows with kept first tokens, sinks and distance penalties with peaked scores at head sizes 32, 64 and 128,
    where bfloat16 prompts run on tiles of 64 queries by 128 keys and single tokens on split keys: prompts of 300
    tokens (windows that straddle a key tile's and a page's border, kept tokens that fill more than a tile), portions
    of many sizes, decoding, and a mixed batch."""
    cfg, d = getattr(sc, name), dirs(name)
    reqs = sc.requests(cfg["vocab"], [300, 130, 64, 7], seed=25)
    mixed, _ = ru.trace_mixed(reqs, seed=8, max_live=4, tail=6)
    for label, steps in (("whole", ru.trace_whole(reqs)), ("decode", ru.trace_decode_tail(reqs, tail=30)),
                         ("chunks", ru.trace_chunks(reqs, seed=5, sizes=(2, 70, 3, 129, 16, 64))), ("mixed", mixed)):
        runner = _runner(d, dtype, n_pages=-(-ru.peak_tokens(steps) // 16) + 4, page=16)
        sc.check_against_plain(d, reqs, steps, ru.run_in_process(runner, steps), dtype, cfg["vocab"], f"{name} {label}")


@pytest.mark.parametrize("page", [4, 16])
def test_far_keys_among_hundreds(dirs, page):
    """An attention that sees every key, a window of 300 keys that keeps the first 40, and heads whose distance penalty
    is slight, all with peaked scores: a key far back that is lost (a page of the table, a window that ends early, a
    kept token) changes whole rows."""
    cfg, d = sc.PEAKED_FAR, dirs("PEAKED_FAR")
    reqs = sc.requests(cfg["vocab"], [400, 200], seed=23)
    for label, steps in (("whole", ru.trace_whole(reqs)), ("decode", ru.trace_decode_tail(reqs, tail=40)),
                         ("chunks", ru.trace_chunks(reqs, seed=4, sizes=(2, 70, 3, 129, 16)))):
        runner = _runner(d, "float32", n_pages=-(-ru.peak_tokens(steps) // page), page=page)
        sc.check_against_plain(d, reqs, steps, ru.run_in_process(runner, steps), "float32", cfg["vocab"], f"far keys page {page} {label}",
                               tol=sc.TOL_PEAKED)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_prompt_of_a_thousand_tokens(dirs, dtype):
    """One prompt of 1,100 tokens whole, in portions of hundreds and of two tokens, and with its last tokens one by
    one: many key tiles, block tables of dozens of pages, pages that a window has passed, kept pages that stay."""
    cfg, d = sc.LARGER, dirs("LARGER")
    reqs = sc.requests(cfg["vocab"], [1100], seed=81)
    for label, steps in (("whole", ru.trace_whole(reqs)), ("chunks", ru.trace_chunks(reqs, seed=8, sizes=(300, 2, 129, 64, 401))),
                         ("decode", ru.trace_decode_tail(reqs, tail=25))):
        runner = _runner(d, dtype, n_pages=ru.peak_tokens(steps) // 16, page=16)
        sc.check_against_plain(d, reqs, steps, ru.run_in_process(runner, steps), dtype, cfg["vocab"], f"long prompt {label}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding_and_slots_used_again(dirs, dtype):
    """One state slot and a small pool: three requests one after the other, each a short prompt and then 150
    tokens one by one, every one of them compared; the slot and the pages are the same ones each time."""
    cfg, d = sc.MIXED_A, dirs("MIXED_A")
    reqs = sc.requests(cfg["vocab"], [153, 151, 152], seed=31)
    steps = ru.trace_decode_tail(reqs, tail=150)
    runner = _runner(d, dtype, n_pages=40, max_num_seqs=1)
    sc.check_against_plain(d, reqs, steps, ru.run_in_process(runner, steps), dtype, cfg["vocab"], "long decoding")
    assert runner.check() == "" and runner.info()["free_pages"] == 40


def test_batches_of_unequal_requests_equal_each_alone(dirs):
    """The logits of a position do not depend on what else is in the batch, beyond rounding: the mixed family's
    rows against the same requests run whole and alone, engine against engine, in bfloat16."""
    cfg, d = sc.MIXED_B, dirs("MIXED_B")
    reqs = sc.requests(cfg["vocab"], [3, 50, 18, 64, 7], seed=41)
    fam = _families(reqs, seed=4)
    got = {}
    for family in ("whole", "mixed"):
        runner = _runner(d, "bfloat16", n_pages=ru.peak_tokens(fam[family]) // 4)
        got[family] = ru.collect(fam[family], ru.run_in_process(runner, fam[family]), cfg["vocab"])
    errs = sorted(sc.row_error(got["mixed"][r][p], got["whole"][r][p].astype(np.float64)) for r in reqs for p in range(len(reqs[r])))
    print(f"mixed against alone, bfloat16: worst {errs[-1]:.3e}, second {errs[-2]:.3e}")
    # (a router's close call may fall the other way in one row; no second row may differ that much)
    assert errs[-2] <= 2e-2 and errs[-1] <= 0.2


def test_residual_stream_after_every_layer(dirs):
    """Layer by layer: models that stop after 1, 2, ... layers of MIXED_A's list agree with the plain model's
    logits, so a fault is pinned to the first layer that shows it."""
    from mini_llm_amd import write_random_model
    import tempfile
    full = sc.MIXED_A
    for n in range(1, len(full["layers"]) + 1):
        cfg = copy.deepcopy(full)
        cfg["layers"] = cfg["layers"][:n]
        with tempfile.TemporaryDirectory() as d:
            write_random_model(cfg, d, 9)
            reqs = sc.requests(cfg["vocab"], [21], seed=n)
            steps = ru.trace_chunks(reqs, seed=n, sizes=(5, 2, 9))
            runner = _runner(d, "float32", n_pages=16)
            sc.check_against_plain(d, reqs, steps, ru.run_in_process(runner, steps), "float32", cfg["vocab"], f"first {n} layers")
            pc, pw = ps.read_model(d)
            assert ps.streams(pc, pw, reqs["r0"]).shape[0] == n


@pytest.mark.parametrize("dtype", DTYPES)
def test_trace_run_program(dirs, tmp_path, dtype):
    """The mixed family through bin/trace_run as a user drives it (its default page size and four state slots)."""
    cfg, d = sc.MIXED_A, dirs("MIXED_A")
    reqs = sc.requests(cfg["vocab"], [2, 33, 64, 5, 70, 21], seed=51)
    steps, _ = ru.trace_mixed(reqs, seed=5, max_live=4, tail=5)
    out = ru.run_trace_run(d, dtype, steps, str(tmp_path / "out"), ru.peak_tokens(steps))
    sc.check_against_plain(d, reqs, steps, out, dtype, cfg["vocab"], "program mixed")


@pytest.mark.parametrize("dtype", DTYPES)
def test_greedy_generation_through_the_engine(dirs, dtype):
    """Engine.generate (scheduler, continuous batching, prompt portions of 7 tokens, two requests at a time for
    five prompts, pages of 4) against the plain model's greedy tokens."""
    from mini_llm_amd import Engine, EngineOptions, SamplingParams
    cfg_d, d = sc.MIXED_A, dirs("MIXED_A")
    cfg, w = ps.read_model(d)
    prompts = list(sc.requests(cfg_d["vocab"], [1, 6, 19, 30, 11], seed=61).values())
    engine = Engine.from_pretrained(d, dtype=dtype, options=EngineOptions(kv_block_size=4, total_kv_blocks=64, max_batch_num=2,
                                                                          max_tokens_per_step=16, prefill_chunk=7))
    outs = engine.generate(prompts, SamplingParams(max_new_tokens=9, ignore_eos=True))
    for p, o in zip(prompts, outs):
        assert len(o) == 9
        if dtype == "float32":
            assert o == ps.greedy_generate(cfg, w, p, 9)
        else:
            # bfloat16 may turn a near-tie: every token must be one the plain model chose or nearly chose
            ids = list(p)
            for t in o:
                row = ps.logits(cfg, w, ids)[-1]
                assert float(row[t]) >= float(row.max()) - 0.08 * float(row.std()), (o, t)
                ids.append(t)
