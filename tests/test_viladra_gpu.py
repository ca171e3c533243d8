"""Viladra through the engine on the GPU against the plain implementation (tests/plain_viladra.py), in 32-bit
and in bfloat16: each mechanism alone, whole prompts against token-by-token decoding, portions down to two
tokens, mixed batches against each request alone, pages and state slots that are used again, keys at window
and page borders and far back, the first tokens, long decoding, and greedy generation through the engine's own
entry point and scheduler."""
import copy

import numpy as np
import pytest

import plain_viladra as pv
import replay_util as ru
import viladra_cases as vc

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]


@pytest.fixture(scope="module")
def dirs(tmp_path_factory):
    from mini_llm_amd import write_random_model
    made = {}

    def get(name, seed=3):
        if name not in made:
            d = tmp_path_factory.mktemp("viladra_" + name)
            write_random_model(dict(getattr(vc, name)), str(d), seed)
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
@pytest.mark.parametrize("name", ["ONLY_RETENTION", "ONLY_RETENTION_PLAIN", "ONLY_GLA", "ONLY_GLA_WIDE", "ONLY_ATTENTION",
                                  "ONLY_ATTENTION_SQUARE", "ONLY_EXPERTS", "ONLY_EXPERTS_ALL", "ONE_EXPERT", "NO_CONVOLUTION"])
def test_each_mechanism_alone(dirs, name, dtype):
    cfg, d = getattr(vc, name), dirs(name)
    reqs = vc.requests(cfg["vocab"], [1, 2, 3, 9, 37, 64, 65, 150], seed=5)
    for label, steps in (("whole", ru.trace_whole(reqs)), ("chunks", ru.trace_chunks(reqs, seed=1)),
                         ("decode", ru.trace_decode_tail(reqs, tail=20))):
        runner = _runner(d, dtype, n_pages=ru.peak_tokens(steps) // 4)
        vc.check_against_plain(d, reqs, steps, ru.run_in_process(runner, steps), dtype, cfg["vocab"], f"{name} {label}")
        assert runner.check() == "" and runner.info()["n_requests"] == 0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["MIXED_A", "MIXED_B", "ODD"])
@pytest.mark.parametrize("family", ["whole", "decode", "chunks", "mixed"])
def test_schedule_families_match_plain(dirs, name, family, dtype):
    """Each request whole; most of it at once and the rest token by token; portions down to two tokens; up to
    four live requests in mixed batches. The pool holds just the peak of live tokens and there are four state
    slots for eight requests, so pages and slots are used again (and were filled with NaN before)."""
    cfg, d = getattr(vc, name), dirs(name)
    reqs = vc.requests(cfg["vocab"], [1, 2, 3, 4, 5, 29, 64, 71] + ([150] if name == "ODD" else []), seed=11)
    steps = _families(reqs, seed=2)[family]
    n_pages = ru.peak_tokens(steps) // 4
    runner = _runner(d, dtype, n_pages)
    vc.check_against_plain(d, reqs, steps, ru.run_in_process(runner, steps), dtype, cfg["vocab"], f"{name} {family}")
    info = runner.info()
    assert runner.check() == "" and info["free_pages"] == n_pages and info["n_requests"] == 0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("page", [8, 16, 64])
@pytest.mark.parametrize("family", ["whole", "decode", "chunks", "mixed"])
def test_sizes_of_a_larger_models_layers(dirs, family, page, dtype):
    """Heads of 64 and 128 at pages of 8 to 64 tokens; prompts of up to 300 tokens (several key tiles, windows that
    end inside a tile, many chunks of the scan), portions, and mixed batches whose single tokens ride along."""
    cfg, d = vc.LARGER, dirs("LARGER")
    reqs = vc.requests(cfg["vocab"], [1, 2, 17, 63, 64, 65, 130, 300], seed=71)
    steps = _families(reqs, seed=6)[family]
    runner = _runner(d, dtype, n_pages=-(-ru.peak_tokens(steps) // page), page=page)
    vc.check_against_plain(d, reqs, steps, ru.run_in_process(runner, steps), dtype, cfg["vocab"], f"larger page {page} {family}")
    assert runner.check() == "" and runner.info()["n_requests"] == 0


@pytest.mark.parametrize("page", [2, 4, 16])
def test_window_and_page_borders_with_peaked_scores(dirs, page):
    """Scores scaled so that single keys dominate, windows of 5 and 16 over pages of 2, 4 and 16 tokens: a window
    that is one key off, or a key lost at a page's border, changes whole rows. Prompts, portions that start and
    end inside a window, and decoding."""
    cfg, d = vc.PEAKED, dirs("PEAKED")
    reqs = vc.requests(cfg["vocab"], [40, 23, 17], seed=21)
    for label, steps in (("whole", ru.trace_whole(reqs)), ("decode", ru.trace_decode_tail(reqs, tail=19)),
                         ("chunks", ru.trace_chunks(reqs, seed=3, sizes=(2, 5, 3, 16, 7, 2, 4)))):
        runner = _runner(d, "float32", n_pages=-(-ru.peak_tokens(steps) // page), page=page)
        vc.check_against_plain(d, reqs, steps, ru.run_in_process(runner, steps), "float32", cfg["vocab"], f"peaked page {page} {label}",
                               tol=vc.TOL_PEAKED)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["PEAKED_TILES_32", "PEAKED_TILES_64", "PEAKED_TILES_128"])
def test_window_borders_at_the_tiled_kernels_head_sizes(dirs, name, dtype):
    """Small windows with peaked scores at head sizes 32, 64 and 128, where bfloat16 prompts run on tiles of 64
    queries by 128 keys and single tokens on split keys: prompts of 300 tokens (windows that straddle a key tile's
    and a page's border), portions of many sizes, decoding, and a mixed batch. The plain model with the window one
    key wider fails the same comparison by far."""
    cfg, d = getattr(vc, name), dirs(name)
    reqs = vc.requests(cfg["vocab"], [300, 130, 64, 7], seed=25)
    mixed, _ = ru.trace_mixed(reqs, seed=8, max_live=4, tail=6)
    for label, steps in (("whole", ru.trace_whole(reqs)), ("decode", ru.trace_decode_tail(reqs, tail=30)),
                         ("chunks", ru.trace_chunks(reqs, seed=5, sizes=(2, 70, 3, 129, 16, 64))), ("mixed", mixed)):
        runner = _runner(d, dtype, n_pages=-(-ru.peak_tokens(steps) // 16) + 4, page=16)
        vc.check_against_plain(d, reqs, steps, ru.run_in_process(runner, steps), dtype, cfg["vocab"], f"{name} {label}")
    if dtype == "bfloat16":
        c, w = pv.read_model(d)
        wider = copy.deepcopy(c)
        wider["layers"][0]["mixer"]["mask"]["size"] += 1
        toks = reqs["r0"]
        a, b = pv.forward(c, w, toks).numpy(), pv.forward(wider, w, toks).numpy()
        errs = np.array([vc.row_error(b[p], a[p]) for p in range(10, len(toks))])
        assert (errs > 3 * vc.TOL["bfloat16"]).mean() > 0.25, errs


@pytest.mark.parametrize("page", [4, 16])
def test_far_keys_among_hundreds(dirs, page):
    """A window of 300 keys with peaked scores, a recurrence that never forgets and ones that forget slowly: a key
    far back that is lost (a page of the table, a window that ends early, a chunk's state) changes whole rows."""
    cfg, d = vc.PEAKED_FAR, dirs("PEAKED_FAR")
    reqs = vc.requests(cfg["vocab"], [400, 200], seed=23)
    for label, steps in (("whole", ru.trace_whole(reqs)), ("decode", ru.trace_decode_tail(reqs, tail=40)),
                         ("chunks", ru.trace_chunks(reqs, seed=4, sizes=(2, 70, 3, 129, 16)))):
        runner = _runner(d, "float32", n_pages=-(-ru.peak_tokens(steps) // page), page=page)
        vc.check_against_plain(d, reqs, steps, ru.run_in_process(runner, steps), "float32", cfg["vocab"], f"far keys page {page} {label}",
                               tol=vc.TOL_PEAKED)


@pytest.mark.parametrize("what", ["window", "first_token", "decay"])
def test_the_peaked_cases_have_teeth(dirs, what):
    """The plain model with every window one key wider, with a sequence's first token changed, or with one decay a
    little off differs from the plain model by far more than the tolerance, in most late rows: the tests above
    would show a window's edge, a lost far token or a wrong decay."""
    name = "PEAKED" if what == "window" else "PEAKED_FAR"
    d = dirs(name)
    cfg, w = pv.read_model(d)
    n = 40 if what == "window" else 330
    toks = vc.requests(cfg["vocab"], [n], seed=21)["r0"]
    a = pv.forward(cfg, w, toks).numpy()
    off, toks_b = copy.deepcopy(cfg), list(toks)
    if what == "window":
        for l in off["layers"]:
            l["mixer"]["mask"]["size"] += 1
    elif what == "first_token":
        toks_b[0] = (toks_b[0] + 1) % cfg["vocab"]
    else:
        off["layers"][1]["mixer"]["decay"][1] = 0.99
    b = pv.forward(off, w, toks_b).numpy()
    late = range(8, n) if what == "window" else range(n - 30, n)
    errs = np.array([vc.row_error(b[p], a[p]) for p in late])
    assert (errs > 20 * vc.TOL_PEAKED).mean() > 0.8, errs


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_prompt_of_a_thousand_tokens(dirs, dtype):
    """One prompt of 1,100 tokens whole, in portions of hundreds and of two tokens, and with its last tokens one by
    one: many key tiles, many chunks of the scan, block tables of dozens of pages, pages that a window has passed."""
    cfg, d = vc.LARGER, dirs("LARGER")
    reqs = vc.requests(cfg["vocab"], [1100], seed=81)
    for label, steps in (("whole", ru.trace_whole(reqs)), ("chunks", ru.trace_chunks(reqs, seed=8, sizes=(300, 2, 129, 64, 401))),
                         ("decode", ru.trace_decode_tail(reqs, tail=25))):
        runner = _runner(d, dtype, n_pages=ru.peak_tokens(steps) // 16, page=16)
        vc.check_against_plain(d, reqs, steps, ru.run_in_process(runner, steps), dtype, cfg["vocab"], f"long prompt {label}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding_and_slots_used_again(dirs, dtype):
    """One state slot and a small pool: three requests one after the other, each a short prompt and then 150
    tokens one by one, every one of them compared; the slot and the pages are the same ones each time."""
    cfg, d = vc.MIXED_A, dirs("MIXED_A")
    reqs = vc.requests(cfg["vocab"], [153, 151, 152], seed=31)
    steps = ru.trace_decode_tail(reqs, tail=150)
    runner = _runner(d, dtype, n_pages=40, max_num_seqs=1)
    vc.check_against_plain(d, reqs, steps, ru.run_in_process(runner, steps), dtype, cfg["vocab"], "long decoding")
    assert runner.check() == "" and runner.info()["free_pages"] == 40


def test_batches_of_unequal_requests_equal_each_alone(dirs):
    """The logits of a position do not depend on what else is in the batch, beyond rounding: the mixed family's
    rows against the same requests run whole and alone, engine against engine, in bfloat16."""
    cfg, d = vc.MIXED_B, dirs("MIXED_B")
    reqs = vc.requests(cfg["vocab"], [3, 50, 18, 64, 7], seed=41)
    fam = _families(reqs, seed=4)
    got = {}
    for family in ("whole", "mixed"):
        runner = _runner(d, "bfloat16", n_pages=ru.peak_tokens(fam[family]) // 4)
        got[family] = ru.collect(fam[family], ru.run_in_process(runner, fam[family]), cfg["vocab"])
    errs = sorted(vc.row_error(got["mixed"][r][p], got["whole"][r][p].astype(np.float64)) for r in reqs for p in range(len(reqs[r])))
    print(f"mixed against alone, bfloat16: worst {errs[-1]:.3e}, second {errs[-2]:.3e}")
    # (a router's close call may fall the other way in one row; no second row may differ that much)
    assert errs[-2] <= 2e-2 and errs[-1] <= 0.2


def test_residual_stream_after_every_layer(dirs):
    """Layer by layer: models that stop after 1, 2, ... layers of MIXED_A's list agree with the plain model's
    logits, so a fault is pinned to the first layer that shows it; and the plain model's streams are what its
    logits are made of."""
    from mini_llm_amd import write_random_model
    import tempfile
    full = vc.MIXED_A
    for n in range(1, len(full["layers"]) + 1):
        cfg = copy.deepcopy(full)
        cfg["layers"] = cfg["layers"][:n]
        with tempfile.TemporaryDirectory() as d:
            write_random_model(cfg, d, 9)
            reqs = vc.requests(cfg["vocab"], [21], seed=n)
            steps = ru.trace_chunks(reqs, seed=n, sizes=(5, 2, 9))
            runner = _runner(d, "float32", n_pages=16)
            vc.check_against_plain(d, reqs, steps, ru.run_in_process(runner, steps), "float32", cfg["vocab"], f"first {n} layers")
            pc, pw = pv.read_model(d)
            handed, last = pv.streams(pc, pw, reqs["r0"])
            assert handed.shape[0] == n and bool((handed[-1] == last).all())


@pytest.mark.parametrize("dtype", DTYPES)
def test_trace_run_program(dirs, tmp_path, dtype):
    """The mixed family through bin/trace_run as a user drives it (its default page size and four state slots)."""
    cfg, d = vc.MIXED_A, dirs("MIXED_A")
    reqs = vc.requests(cfg["vocab"], [2, 33, 64, 5, 70, 21], seed=51)
    steps, _ = ru.trace_mixed(reqs, seed=5, max_live=4, tail=5)
    out = ru.run_trace_run(d, dtype, steps, str(tmp_path / "out"), ru.peak_tokens(steps))
    vc.check_against_plain(d, reqs, steps, out, dtype, cfg["vocab"], "program mixed")


@pytest.mark.parametrize("dtype", DTYPES)
def test_greedy_generation_through_the_engine(dirs, dtype):
    """Engine.generate (scheduler, continuous batching, prompt portions of 7 tokens, two requests at a time for
    five prompts, pages of 4) against the plain model's greedy tokens."""
    from mini_llm_amd import Engine, EngineOptions, SamplingParams
    cfg_d, d = vc.MIXED_A, dirs("MIXED_A")
    cfg, w = pv.read_model(d)
    prompts = list(vc.requests(cfg_d["vocab"], [1, 6, 19, 30, 11], seed=61).values())
    engine = Engine.from_pretrained(d, dtype=dtype, options=EngineOptions(kv_block_size=4, total_kv_blocks=64, max_batch_num=2,
                                                                          max_tokens_per_step=16, prefill_chunk=7))
    outs = engine.generate(prompts, SamplingParams(max_new_tokens=9, ignore_eos=True))
    for p, o in zip(prompts, outs):
        assert len(o) == 9
        if dtype == "float32":
            assert o == pv.greedy_generate(cfg, w, p, 9)
        else:
            # bfloat16 may turn a near-tie: every token must be one the plain model chose or nearly chose
            ids = list(p)
            for t in o:
                row = pv.forward(cfg, w, ids)[-1]
                assert float(row[t]) >= float(row.max()) - 0.08 * float(row.std()), (o, t)
                ids.append(t)
