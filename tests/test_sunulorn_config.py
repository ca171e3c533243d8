"""Sunulorn without a GPU: what its configuration asks of a checkpoint, what it refuses, the plain implementation's
own consistency (closed forms of the single mechanisms), that the peaked cases of the GPU tests would show a mask,
sink or slope that is off, and the cache manager's kept first pages."""
import copy
import math

import pytest
import torch

import plain_sunulorn as ps
import sunulorn_cases as sc
from mini_llm_amd import check_model_dir, describe_config, registered_architectures, write_random_model
from mini_llm_amd.config import ConfigError


def test_registered_and_tensors_follow_the_layer_list():
    assert "Sunulorn" in registered_architectures()
    d = describe_config(sc.MIXED_A)
    assert d["architecture"] == "Sunulorn"
    shapes = {t["name"]: t["shape"] for t in d["tensors"]}
    assert shapes["embed"] == [257, 64] and shapes["head"] == [257, 64] and shapes["final.norm"] == [64]
    # attention_3: biases on queries, keys and values, one gate row and one sink per head, no bias behind the output
    assert shapes["l0.mix.q"] == [64, 64] and shapes["l0.mix.k"] == [32, 64] and shapes["l0.mix.v.b"] == [32]
    assert shapes["l0.mix.sink"] == [4] and shapes["l0.mix.g"] == [4, 64] and "l0.mix.o.b" not in shapes
    # attention: no biases, no values, taps on queries and keys
    assert shapes["l1.mix.q.conv"] == [64, 3] and shapes["l1.mix.k.conv"] == [32, 3]
    assert "l1.mix.v" not in shapes and "l1.mix.q.b" not in shapes and "l1.mix.g" not in shapes and shapes["l1.mix.o"] == [64, 64]
    # attention_2: values of a width of their own, a gate per output column, a bias behind the output
    assert shapes["l2.mix.v"] == [48, 64] and shapes["l2.mix.g"] == [96, 64] and shapes["l2.mix.o"] == [64, 96] and shapes["l2.mix.o.b"] == [64]
    # a layer that reads another's keys and values has no projections for them
    assert "l3.mix.k" not in shapes and "l3.mix.v.b" not in shapes and shapes["l3.mix.q.b"] == [64] and shapes["l3.mix.sink"] == [4]
    # no feed-forward: no second norm; dense and routed feed-forwards
    assert "l3.norm2" not in shapes and "l3.mlp.gate" not in shapes
    assert shapes["l1.mlp.gate"] == [40, 64] and shapes["l1.mlp.down"] == [64, 40]
    assert shapes["l2.mlp.e5.gate"] == [16, 64] and shapes["l2.mlp.e5.down"] == [64, 16] and "l2.mlp.e6.up" not in shapes
    assert shapes["l2.mlp.router"] == [6, 64] and shapes["l2.mlp.shared.sg"] == [1, 64] and shapes["l2.mlp.shared.up"] == [24, 64]
    assert "l4.mlp.shared.sg" not in shapes and "l4.mlp.shared.up" not in shapes
    roles = {t["name"]: t["role"] for t in d["tensors"]}
    assert roles["l2.mlp.router"] == "matrix" and roles["l1.mix.q.conv"] == "vector" and roles["l0.mix.sink"] == "vector"


def test_keys_that_may_be_absent_have_the_plain_meaning():
    cfg = copy.deepcopy(sc.MIXED_A)
    m = cfg["layers"][2]["mixer"]
    heads, dim = m["heads"], m["dim"]
    m.pop("kv_heads"); m.pop("vdim"); m.pop("mask"); m.pop("rot")
    cfg["layers"][1]["mlp"].pop("kind")          # dense
    cfg["layers"][1]["mixer"].pop("conv")
    cfg["layers"][4]["mixer"]["conv"] = 0            # (no taps: no convolution either)
    cfg.pop("embedding")
    shapes = {t["name"]: t["shape"] for t in describe_config(cfg)["tensors"]}
    assert shapes["l2.mix.k"] == [heads * dim, 64] and shapes["l2.mix.v"] == [heads * dim, 64]
    assert "l1.mlp.gate" in shapes and "l1.mix.q.conv" not in shapes and "l4.mix.k.conv" not in shapes


@pytest.mark.parametrize("change, message", [
    (lambda c: c["layers"][1].__setitem__("type", "lstm"), "unknown layer type"),
    (lambda c: c["layers"][1]["mixer"].__setitem__("kv_heads", 3), "multiple of kv_heads"),
    (lambda c: c["layers"][1]["mixer"]["rot"].__setitem__("dims", 3), "even"),
    (lambda c: c["layers"][1]["mixer"]["rot"].__setitem__("dims", 18), "at most dim"),
    (lambda c: c["layers"][1]["mixer"].__setitem__("vdim", 8), "vdim must equal dim"),
    (lambda c: c["layers"][1]["mixer"].__setitem__("conv", 17), "16 taps"),
    (lambda c: c["layers"][3]["mixer"].__setitem__("kv_from", 3), "earlier layer"),
    (lambda c: c["layers"][3]["mixer"].__setitem__("kv_from", 1), "attention_3 layer"),
    (lambda c: c["layers"][5]["mixer"].__setitem__("kv_from", 3), "keys and values of its own"),
    (lambda c: c["layers"][3]["mixer"].__setitem__("dim", 8), "must equal those"),
    (lambda c: c["layers"][0]["mlp"]["router"].__setitem__("top", 9), "top"),
    (lambda c: c["layers"][0]["mlp"]["expert"].__setitem__("limit", 0.0), "limit"),
    (lambda c: c["layers"][0]["mlp"].__setitem__("kind", "mystery"), "dense"),
    (lambda c: c["layers"][2]["mixer"].pop("scale"), "scale"),
    (lambda c: c.pop("norm"), "norm"),
])
def test_refusals(change, message):
    cfg = copy.deepcopy(sc.MIXED_A)
    change(cfg)
    with pytest.raises(ConfigError, match=message):
        describe_config(cfg)


def test_written_folder_checks(tmp_path):
    d = write_random_model(dict(sc.MIXED_B), str(tmp_path / "m"), 1)
    arch, n_tensors, _ = check_model_dir(d)
    assert arch == "Sunulorn" and n_tensors == len(describe_config(sc.MIXED_B)["tensors"])
    cfg, w = ps.read_model(d)
    assert ps.logits(cfg, w, [1, 2, 3, 4, 5]).shape == (5, 513)


# -- the plain mechanisms against closed forms -----------------------------------------------------------
def test_convolution_last_tap_is_the_tokens_own():
    u = torch.arange(12, dtype=torch.float64).view(6, 2) + 1
    taps = torch.tensor([[0.0, 0.0, 1.0], [1.0, 0.0, 0.0]], dtype=torch.float64)
    y = ps.causal_convolution(u, taps)
    assert torch.equal(y[:, 0], u[:, 0])                                             # only the last tap: the input itself
    assert torch.equal(y[2:, 1], u[:-2, 1]) and float(y[:2, 1].abs().sum()) == 0     # only the first tap: two tokens back, zeros in front


def test_turns_keep_lengths_and_pair_the_right_columns():
    v = torch.randn(5, 2, 8, dtype=torch.float64)
    pos = [0, 1, 2, 30, 400]
    for turn in (ps.turn_interleaved, ps.turn_half_split):
        out = turn(v, pos, 100.0, 6)
        assert torch.allclose(out.norm(dim=-1), v.norm(dim=-1)) and torch.equal(out[..., 6:], v[..., 6:]) and torch.equal(out[0], v[0])
    one = torch.zeros(1, 1, 8, dtype=torch.float64)
    one[0, 0, 2] = 1.0
    a = 3 * 100.0 ** (-2.0 / 6)                     # position 3, pair 1
    il = ps.turn_interleaved(one, [3], 100.0, 6)[0, 0]
    assert math.isclose(float(il[2]), math.cos(a)) and math.isclose(float(il[3]), math.sin(a)) and float(il[5]) == 0
    one.zero_(); one[0, 0, 1] = 1.0
    hs = ps.turn_half_split(one, [3], 100.0, 6)[0, 0]
    assert math.isclose(float(hs[1]), math.cos(a)) and math.isclose(float(hs[4]), math.sin(a)) and float(hs[2]) == 0


def test_visible_window_with_kept_first_tokens():
    see = ps.visible(12, {"size": 3, "keep_first": 2})
    assert [j for j in range(12) if see[9, j]] == [0, 1, 7, 8, 9]
    assert [j for j in range(12) if see[2, j]] == [0, 1, 2] and [j for j in range(12) if see[3, j]] == [0, 1, 2, 3]
    assert bool(ps.visible(5, None)[4, 0]) and not bool(ps.visible(5, None)[0, 1])


def test_softmax_with_sink_and_slope_closed_form():
    # one head, equal keys: the weights follow the distance penalty alone, and the sink takes its share
    T = 4
    q = torch.ones(T, 1, 2, dtype=torch.float64)
    k = torch.ones(T, 1, 2, dtype=torch.float64)
    v = torch.eye(T, dtype=torch.float64).view(T, 1, T)
    out = ps.softmax_attention(q, k, v, 0.5, slopes=[0.25], sink=torch.tensor([0.7], dtype=torch.float64))
    e = [math.exp(1.0 - 0.25 * dist) for dist in range(T)]
    denom = sum(e) + math.exp(0.7)
    assert torch.allclose(out[3, 0], torch.tensor([e[3], e[2], e[1], e[0]], dtype=torch.float64) / denom)
    no_sink = ps.softmax_attention(q, k, v, 0.5)
    assert math.isclose(float(no_sink[3, 0].sum()), 1.0) and float(out[3, 0].sum()) < 1.0
    assert ps.head_slopes(4) == [0.25, 0.0625, 0.015625, 0.00390625]


def test_expert_weight_stands_on_the_input():
    w = {"e.gate": torch.tensor([[2.0, 0.0]], dtype=torch.float64), "e.up": torch.tensor([[0.0, 4.0]], dtype=torch.float64),
         "e.down": torch.tensor([[1.0], [0.0]], dtype=torch.float64)}
    h = torch.tensor([[1.0, 1.0]], dtype=torch.float64)
    y = ps.clamped_expert(0.25 * h, w, "e.", 0.75)
    g, u = 0.5, 0.75                                # gate below the limit, up clamped to it
    assert math.isclose(float(y[0, 0]), g / (1 + math.exp(-1.702 * g)) * (u + 1)) and float(y[0, 1]) == 0
    assert ps.chosen_experts(torch.tensor([[0.2, 0.9, 0.9, 0.1]]), 2) == [[1, 2]]


@pytest.mark.parametrize("what", ["window", "keep_first", "first_token", "sink", "slope", "zero_sink"])
def test_the_peaked_cases_have_teeth(tmp_path, what):
    """The plain model with a window one key wider, one kept token fewer, a sequence's first token changed, a sink
    left out or a slope a little off differs from the plain model by far more than the tolerance in many late rows:
    the GPU tests would show such a fault."""
    name = "PEAKED_FAR" if what == "first_token" else "SINK_SOFT" if what in ("sink", "zero_sink") else "PEAKED"
    d = write_random_model(dict(getattr(sc, name)), str(tmp_path / "m"), 3)
    cfg, w = ps.read_model(d)
    n = 330 if what == "first_token" else 40
    toks = sc.requests(cfg["vocab"], [n], seed=21)["r0"]
    a = ps.logits(cfg, w, toks).numpy()
    off, toks_b, w_b = copy.deepcopy(cfg), list(toks), dict(w)
    if what == "window":
        for l in off["layers"][:2]:
            l["mixer"]["mask"]["size"] += 1
    elif what == "keep_first":
        for l in off["layers"][:2]:
            l["mixer"]["mask"]["keep_first"] -= 1
    elif what == "first_token":
        toks_b[0] = (toks_b[0] + 1) % cfg["vocab"]
    elif what == "sink":
        w_b["l1.mix.sink"] = torch.full_like(w["l1.mix.sink"], -50.0)
    elif what == "slope":
        orig = ps.head_slopes
        ps.head_slopes = lambda H: [s * 1.5 for s in orig(H)]
    try:
        if what == "zero_sink":
            # the 'attention' layer's own extra term: the plain model without it
            orig_mixer = ps.conv_attention_mixer
            orig_attn = ps.softmax_attention
            ps.softmax_attention = lambda *args, **kw: orig_attn(*args, **{k: v for k, v in kw.items() if k != "sink" or v.abs().sum() != 0})
        b = ps.logits(off, w_b, toks_b).numpy()
    finally:
        if what == "slope":
            ps.head_slopes = orig
        if what == "zero_sink":
            ps.softmax_attention = orig_attn
    late = range(n - 30, n)
    errs = [sc.row_error(b[p], a[p]) for p in late]
    floor = 20 * (sc.TOL["float32"] if name == "SINK_SOFT" else sc.TOL_PEAKED)
    assert sum(e > floor for e in errs) > 0.5 * len(errs), errs


def test_cache_manager_keeps_the_first_pages_of_a_window_group():
    from mini_llm_amd.cache.manager import CacheManager, GroupSpec
    m = CacheManager([GroupSpec(page_size=4, n_pages=32, window=8, keep_first=6)], n_state_slots=2)
    assert m.add_request(1) >= 0
    m.reserve(1, 40)
    m.commit(1, 40)
    table = m.block_table(1, 0)
    held = [b for b, p in enumerate(table) if p >= 0]
    # the next query stands at 40 and reads keys from 33 on: pages 8 and 9; the first 6 keys lie in pages 0 and 1
    assert held == [0, 1, 8, 9], held
    assert m.check() == ""
    m.free_request(1)
    assert m.free_pages(0) == 32 and m.check() == ""
