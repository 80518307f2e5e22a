"""Trace replay on the GPU against the plain implementation: each request alone and whole;
most of it in one step and the last 32 tokens one by one; in portions of changing size;
and mixed, up to four live requests with so few pages that they are used again; in true
32-bit and in bfloat16."""
import json
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest

import schedules
from plain import lfm2 as plain
from replay_common import (BF16_MAX_FACTOR, FP32_TOL, assert_matches_plain, bf16_bounds, collect,
                           first_bad, make_requests, plain_logits, read_outputs, worst_error)
from tiny import TINY, write_tiny

pytestmark = pytest.mark.gpu

ROOT = Path(__file__).resolve().parent.parent
LENGTHS = {"A": [70, 45, 100, 37, 83, 64], "B": [33, 97, 40, 71, 52], "C": [66, 35, 90, 41],
           "D": [50, 81, 36], "E": [45, 70, 33], "F": [66, 40, 85], "G": [70, 38, 51],
           "H": [40, 77, 35]}
MIXED_LENGTHS = {"A": [70, 45, 100, 37, 83, 64, 29, 58, 91, 40],
                 "B": [33, 97, 40, 71, 52, 64, 18, 85, 47],
                 "C": [66, 35, 90, 41, 23, 77, 50, 62],
                 "D": [50, 81, 36, 67, 44, 72, 90, 33, 58, 41],
                 "E": [45, 70, 33, 52, 61, 38, 88, 27, 95, 40],
                 "F": [66, 40, 85, 37, 58, 49, 92, 31, 74, 43],
                 "G": [70, 38, 51, 64, 33, 88, 45, 59, 36, 72],
                 "H": [40, 77, 35, 66, 52, 90, 31, 48, 83, 44]}


@pytest.fixture(scope="module")
def model_dirs(tmp_path_factory):
    base = tmp_path_factory.mktemp("models")
    return {name: write_tiny(name, base / name) for name in TINY}


_models = {}


def gpu_model(model_dir, dtype):
    from kappai_amd.models import load_model
    key = (str(model_dir), dtype)
    if key not in _models:
        _models[key] = load_model(model_dir, dtype, "cuda:0")
    return _models[key]


def replay_in_process(model_dir, dtype, steps, index, max_tokens, out_dir, page_size=16):
    from kappai_amd.engine.replay import TraceReplayer, make_replay_cache
    from kappai_amd.engine.step import StepRunner
    model = gpu_model(model_dir, dtype)
    cache = make_replay_cache(model, max_tokens, page_size)
    cache.allocate_storage(model.dtype, "cuda:0", poison=True)
    rep = TraceReplayer(StepRunner(model, cache, "cuda:0"), out_dir)
    outputs = {}
    for obj in steps:
        res = rep.run_step(obj)
        if res is not None:
            outputs[obj["step"]] = res
    cache.check()
    assert not cache.live_requests()
    return collect(index, outputs, model.vocab_size)


def tolerance(model_dir, requests, dtype):
    """The bound on a single row (tests that look at rows one by one)."""
    if dtype == "float32":
        return FP32_TOL
    keys = [(rid, pos) for rid, toks in requests.items() for pos in range(len(toks))]
    return BF16_MAX_FACTOR * bf16_bounds(model_dir, requests, keys)[0]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E", "F", "G", "H"])
@pytest.mark.parametrize("family", ["whole", "prefill_then_decode", "changing_portions", "mixed"])
def test_schedules(tmp_path, model_dirs, name, family, dtype):
    cfg = TINY[name][0]
    lengths = MIXED_LENGTHS[name] if family == "mixed" else LENGTHS[name]
    requests = make_requests(cfg["vocab_size"], lengths, seed=10)
    steps, index, peak = getattr(schedules, family)(requests)
    got = replay_in_process(model_dirs[name], dtype, steps, index, peak, tmp_path / "out")
    assert len(got) == sum(len(t) for t in requests.values())
    assert_matches_plain(got, model_dirs[name], requests, dtype)


@pytest.mark.parametrize("page_size", [4, 64])
def test_other_page_sizes(tmp_path, model_dirs, page_size):
    cfg = TINY["B"][0]
    requests = make_requests(cfg["vocab_size"], MIXED_LENGTHS["B"], seed=11)
    steps, index, peak = schedules.mixed(requests)
    got = replay_in_process(model_dirs["B"], "float32", steps, index, peak, tmp_path / "out",
                            page_size=page_size)
    ref = plain_logits(model_dirs["B"], requests)
    err, where = worst_error(got, ref)
    assert err < FP32_TOL, (err, where, first_bad(got, ref, FP32_TOL))


def test_long_decoding_and_first_tokens(tmp_path, model_dirs):
    """Two tokens of prompt, then 300 tokens one by one (the first tokens of a sequence, page
    edges, conv history shorter than the taps), two requests side by side."""
    cfg = TINY["B"][0]
    requests = make_requests(cfg["vocab_size"], [302, 301], seed=12)
    plans = {"r0": (0, [2] + [1] * 300), "r1": (0, [1] * 301)}
    steps, index, peak = schedules.build(requests, plans)
    for dtype in ("float32", "bfloat16"):
        got = replay_in_process(model_dirs["B"], dtype, steps, index, peak, tmp_path / dtype)
        assert_matches_plain(got, model_dirs["B"], requests, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_graphs_across_a_context_bucket(tmp_path, model_dirs, dtype):
    """Two requests decoded side by side from position 1000 to 1061, from captured graphs: at
    position 1024 the graphs of the next context bucket take over (wider block tables, other
    key splits) and the rotation tables are built anew at twice their length while graphs that
    read the old ones still exist.  Every logit against the plain implementation."""
    from kappai_amd.engine.replay import TraceReplayer, make_replay_cache
    from kappai_amd.engine.step import StepRunner, _context_bucket
    cfg = TINY["B"][0]
    requests = make_requests(cfg["vocab_size"], [1062, 1040], seed=21)
    plans = {"r0": (0, [1000] + [1] * 62), "r1": (0, [978] + [1] * 62)}
    steps, index, peak = schedules.build(requests, plans, want="last")
    assert _context_bucket(1001) != _context_bucket(1030)
    model = gpu_model(model_dirs["B"], dtype)
    cache = make_replay_cache(model, peak)
    cache.allocate_storage(model.dtype, "cuda:0", poison=True)
    runner = StepRunner(model, cache, "cuda:0")
    rep = TraceReplayer(runner, tmp_path / "out")
    outputs = {}
    for obj in steps:
        res = rep.run_step(obj)
        if res is not None:
            outputs[obj["step"]] = res
    cache.check()
    assert runner.graph_replays >= 50 and len(runner._graphs) >= 2
    got = collect(index, outputs, model.vocab_size)
    assert len(got) == 2 * 63
    assert_matches_plain(got, model_dirs["B"], requests, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(tmp_path, model_dirs, dtype):
    """The program itself, as a user runs it: steps on standard input, 'done <step>' after
    each, <step>.f32 files, exit code 0."""
    cfg = TINY["A"][0]
    requests = make_requests(cfg["vocab_size"], MIXED_LENGTHS["A"][:6], seed=13)
    steps, index, peak = schedules.mixed(requests)
    out = tmp_path / "out"
    proc = subprocess.Popen(
        [sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(model_dirs["A"]),
         "--dtype", dtype, "--out", str(out), "--max-tokens", str(peak)],
        stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True, cwd=str(tmp_path))
    for obj in steps:
        proc.stdin.write(json.dumps(obj) + "\n")
        proc.stdin.flush()
        assert proc.stdout.readline().strip() == f"done {obj['step']}"
    proc.stdin.close()
    assert proc.wait(timeout=120) == 0
    got = collect(index, read_outputs(out, index, cfg["vocab_size"]), cfg["vocab_size"])
    assert_matches_plain(got, model_dirs["A"], requests, dtype)
    # the index beside the files names the same rows: (request, position) in output order
    lines = [json.loads(line) for line in (out / "index.jsonl").read_text().splitlines()]
    assert [ln["step"] for ln in lines] == [s for s, idx in enumerate(index) if idx]
    for ln in lines:
        assert ln["file"] == f"{ln['step']}.f32" and ln["vocab"] == cfg["vocab_size"]
        assert [tuple(r) for r in ln["rows"]] == index[ln["step"]]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_graphs_replay_what_eager_steps_compute(tmp_path, model_dirs, dtype):
    """Steps of single decoded tokens are replayed from captured HIP graphs.  Every replay, with
    eager prompt portions of other requests between them, must give bit for bit what the same
    step gives without graphs."""
    from kappai_amd.engine.replay import TraceReplayer, make_replay_cache
    from kappai_amd.engine.step import StepRunner
    cfg = TINY["B"][0]
    requests = make_requests(cfg["vocab_size"], [40, 44, 91], seed=14)
    plans = {"r0": (0, [10] + [1] * 30), "r1": (0, [14] + [1] * 30),
             "r2": (12, [20, 1, 1, 1, 30, 1, 1, 1, 1, 1, 33])}
    steps, index, peak = schedules.build(requests, plans)
    results = {}
    for graphs in (False, True):
        model = gpu_model(model_dirs["B"], dtype)
        cache = make_replay_cache(model, peak)
        cache.allocate_storage(model.dtype, "cuda:0", poison=True)
        runner = StepRunner(model, cache, "cuda:0", decode_graphs=graphs)
        rep = TraceReplayer(runner, tmp_path / f"g{graphs}")
        results[graphs] = [rep.run_step(obj) for obj in steps]
        assert (runner.graph_replays > 15) == graphs
    for a, b in zip(results[False], results[True]):
        assert (a is None) == (b is None)
        if a is not None:
            assert np.array_equal(a, b)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E", "F", "G", "H"])
def test_steps_from_c_equal_steps_from_the_host(tmp_path, model_dirs, name, dtype):
    """A step is launched by one call into C (kappai_forward) when the model is made of the
    framework's own parts, and part by part from the host otherwise.  Both run the same kernels
    on the same choices: the mixed schedule gives bit for bit the same logits either way, with
    and without decode graphs."""
    from kappai_amd.engine.replay import TraceReplayer, make_replay_cache
    from kappai_amd.engine.step import StepRunner
    cfg = TINY[name][0]
    requests = make_requests(cfg["vocab_size"], MIXED_LENGTHS[name][:7], seed=22)
    steps, index, peak = schedules.mixed(requests)
    results = {}
    for c_forward in (True, False):
        for graphs in (False, True):
            model = gpu_model(model_dirs[name], dtype)
            cache = make_replay_cache(model, peak)
            cache.allocate_storage(model.dtype, "cuda:0", poison=True)
            runner = StepRunner(model, cache, "cuda:0", decode_graphs=graphs, c_forward=c_forward)
            rep = TraceReplayer(runner, tmp_path / f"c{c_forward}g{graphs}")
            results[(c_forward, graphs)] = [rep.run_step(obj) for obj in steps]
            assert (runner._cplan is not None) == c_forward
    base = results[(False, False)]
    for key, res in results.items():
        for a, b in zip(base, res):
            assert (a is None) == (b is None)
            if a is not None:
                assert np.array_equal(a, b), key


# A wider configuration with a long prompt, so that the kernels for large steps run inside the
# engine: the 128 x 128 / 256 x 256 block products (K a multiple of 128, more than 64 rows) and
# the prefill attention that shares key tiles between four heads of a kv head (head size 64,
# 66 q tiles x 4 head quads).
WIDE = {
    "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2",
    "hidden_size": 1024, "num_hidden_layers": 4,
    "layer_types": ["conv", "full_attention", "conv", "full_attention"],
    "num_attention_heads": 16, "num_key_value_heads": 4, "head_dim": 64,
    "intermediate_size": 2688, "block_auto_adjust_ff_dim": False,
    "vocab_size": 2048, "norm_eps": 1e-5, "rope_theta": 1000000.0,
    "conv_L_cache": 3, "conv_bias": False, "tie_embedding": True,
    "max_position_embeddings": 8192,
}


# The same with heads of 128 and eight query heads for every kv head (two groups of four in the
# kernel that shares key tiles; 64 keys a wave and turn in the decode kernel), a head width
# (2048) that is not the model's, and a vocabulary that is no power of two.
WIDE_HEADS = dict(WIDE, hidden_size=512, num_hidden_layers=2,
                  layer_types=["conv", "full_attention"], num_attention_heads=16,
                  num_key_value_heads=2, head_dim=128, intermediate_size=1024, vocab_size=1000,
                  rope_theta=10000.0)


@pytest.mark.parametrize("shape", ["wide", "wide_heads"])
@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_long_prompt_on_a_wide_model(tmp_path, dtype, shape):
    import copy
    from kappai_amd.config import config_from_dict
    from kappai_amd.weights import write_random_model
    WIDE = globals()["WIDE" if shape == "wide" else "WIDE_HEADS"]
    folder = write_random_model(tmp_path / "wide", config_from_dict(copy.deepcopy(WIDE)), seed=5,
                                std=0.02, norm_jitter=0.05)
    requests = make_requests(WIDE["vocab_size"], [2200, 300], seed=15)
    # r0: 66 q tiles in one step, a short portion, then token by token; r1 beside it, cut in two
    plans = {"r0": (0, [2112, 56] + [1] * 32), "r1": (1, [200, 100])}
    steps, index, peak = schedules.build(requests, plans)
    got = replay_in_process(folder, dtype, steps, index, peak, tmp_path / "out")
    assert len(got) == 2500
    assert_matches_plain(got, folder, requests, dtype)


@pytest.mark.parametrize("shape", ["wide", "wide_heads"])
def test_short_portions_on_a_wide_model_from_c_and_from_the_host(tmp_path, shape):
    """Steps of 17 to 256 rows on models wide enough for their in_proj and qkv products to be cut
    into K ranges (portions of 150 and 70 rows beside single decoded tokens, a portion of 40, a
    step of 20 single rows' worth of two requests): the conv and qk-norm kernels add the float
    partial sums up.  Launched from C and part by part from the host the logits are bit for bit
    the same, and both follow the plain implementation."""
    import copy
    from kappai_amd.config import config_from_dict
    from kappai_amd.engine.replay import TraceReplayer, make_replay_cache
    from kappai_amd.engine.step import StepRunner
    from kappai_amd.kernels import ops, tuning
    from kappai_amd.weights import write_random_model
    raw = globals()["WIDE" if shape == "wide" else "WIDE_HEADS"]
    folder = write_random_model(tmp_path / "wide", config_from_dict(copy.deepcopy(raw)), seed=6,
                                std=0.02, norm_jitter=0.05)
    assert ops.split_k_for(150, 3 * raw["hidden_size"], raw["hidden_size"]) > 1      # in_proj is cut
    assert tuning.takes_partial_sums(150, False) and not tuning.takes_partial_sums(300, False)
    requests = make_requests(raw["vocab_size"], [230, 75, 60], seed=16)
    plans = {"r0": (0, [150, 70] + [1] * 10), "r1": (1, [70] + [1] * 5), "r2": (2, [40, 20])}
    steps, index, peak = schedules.build(requests, plans)
    model = gpu_model(folder, "bfloat16")
    results = {}
    for c_forward in (True, False):
        cache = make_replay_cache(model, peak)
        cache.allocate_storage(model.dtype, "cuda:0", poison=True)
        runner = StepRunner(model, cache, "cuda:0", decode_graphs=False, c_forward=c_forward)
        rep = TraceReplayer(runner, tmp_path / f"c{c_forward}")
        outputs = {}
        for obj in steps:
            res = rep.run_step(obj)
            if res is not None:
                outputs[obj["step"]] = res
        cache.check()
        results[c_forward] = outputs
    assert results[True].keys() == results[False].keys()
    for step in results[True]:
        assert np.array_equal(results[True][step], results[False][step]), step
    got = collect(index, results[True], model.vocab_size)
    assert_matches_plain(got, folder, requests, "bfloat16")


def test_decode_attention_with_its_prologue_inside_from_c_and_from_the_host(tmp_path):
    """With more than 512 keys and a head size of 64 a decode step's attention kernel does the
    per-head norm, the rotation and the store of the new key and value itself.  The C side of a
    step and the host's parts must make that choice alike (bit-equal logits), the host's parts
    must have made it (no call of the separate kernel in those steps), and both ways the logits
    stay within the bound of the plain implementation's rounding."""
    import copy
    from kappai_amd.config import config_from_dict
    from kappai_amd.engine.replay import TraceReplayer, make_replay_cache
    from kappai_amd.engine.step import StepRunner
    from kappai_amd.kernels import ops, tuning
    from kappai_amd.weights import write_random_model
    separate = []                    # rows of every call of the kernel that is to be left out
    plain_kernel = ops.qk_norm_rope_store

    def spy(qkv, *args, **kwargs):
        separate.append(qkv.shape[-2])
        return plain_kernel(qkv, *args, **kwargs)

    folder = write_random_model(tmp_path / "wide", config_from_dict(copy.deepcopy(WIDE)), seed=8,
                                std=0.02, norm_jitter=0.05)
    requests = make_requests(WIDE["vocab_size"], [640, 530], seed=17)
    plans = {"r0": (0, [632] + [1] * 8), "r1": (0, [522] + [1] * 8)}
    steps, index, peak = schedules.build(requests, plans, want="last")
    results = {}
    for fused in (True, False):
        for c_forward in (True, False):
            tuning.FUSED_QK = fused
            ops.qk_norm_rope_store = spy
            del separate[:]
            try:
                model = gpu_model(folder, "bfloat16")
                cache = make_replay_cache(model, peak)
                cache.allocate_storage(model.dtype, "cuda:0", poison=True)
                runner = StepRunner(model, cache, "cuda:0", decode_graphs=False,
                                    c_forward=c_forward)
                rep = TraceReplayer(runner, tmp_path / f"f{fused}c{c_forward}")
                outputs = {}
                for obj in steps:
                    res = rep.run_step(obj)
                    if res is not None:
                        outputs[obj["step"]] = res
            finally:
                tuning.FUSED_QK = True
                ops.qk_norm_rope_store = plain_kernel
            if not c_forward:        # two attention layers; one prompt step, eight decode steps
                assert separate == ([1154] * 2 if fused else [1154] * 2 + [2] * 16), separate
            results[(fused, c_forward)] = collect(index, outputs, model.vocab_size)
    for fused in (True, False):
        a, b = results[(fused, True)], results[(fused, False)]
        assert a.keys() == b.keys()
        assert all(np.array_equal(a[k], b[k]) for k in a), fused
        assert_matches_plain(a, folder, requests, "bfloat16")


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_decoded_tokens_over_long_contexts_beside_prompt_portions(tmp_path, dtype, monkeypatch):
    """Two requests decode at more than a thousand tokens of context while a third one's prompt
    runs in portions beside them: in such steps the single rows are listed apart from the tiles
    of the portions and take the decode kernel (bfloat16; float32 runs the plain kernel over
    all rows).  Every logit against the plain implementation, from C and from the host's parts
    bit for bit alike."""
    import copy
    from kappai_amd.config import config_from_dict
    from kappai_amd.engine.replay import TraceReplayer, make_replay_cache
    from kappai_amd.engine.step import StepRunner
    from kappai_amd.weights import write_random_model
    folder = write_random_model(tmp_path / "wide", config_from_dict(copy.deepcopy(WIDE)), seed=9,
                                std=0.02, norm_jitter=0.05)
    from kappai_amd.kernels import tuning
    requests = make_requests(WIDE["vocab_size"], [1100, 1040, 150], seed=18)
    # r0 and r1 whole, then one token a step; r2 arrives later, in portions beside them
    plans = {"r0": (0, [1092] + [1] * 8), "r1": (0, [1032] + [1] * 8), "r2": (2, [70, 2, 45, 33])}
    monkeypatch.setattr(tuning, "LONE_ROWS_FROM", 1024)     # (a thousand tokens get there)
    steps, index, peak = schedules.build(requests, plans, want="last")
    results = {}
    for c_forward in (True, False):
        model = gpu_model(folder, dtype)
        (tiles,) = model.step_tables()
        assert tiles.lone_from == (1024 if dtype == "bfloat16" else None)
        cache = make_replay_cache(model, peak)
        cache.allocate_storage(model.dtype, "cuda:0", poison=True)
        runner = StepRunner(model, cache, "cuda:0", c_forward=c_forward)
        seen = []
        make = runner.make_batch

        def spy(entries, placed=None):
            batch = make(entries, placed)
            lone = batch.extra.get("lone_rows")
            seen.append(None if lone is None else lone.tolist())
            return batch

        runner.make_batch = spy
        rep = TraceReplayer(runner, tmp_path / f"c{c_forward}")
        outputs = {}
        for obj in steps:
            res = rep.run_step(obj)
            if res is not None:
                outputs[obj["step"]] = res
        if dtype == "bfloat16":
            assert [rows for rows in seen if rows is not None] == [[0, 1]] * 4, seen
        else:
            assert all(rows is None for rows in seen)
        results[c_forward] = collect(index, outputs, model.vocab_size)
    assert all(np.array_equal(results[True][k], results[False][k]) for k in results[True])
    assert_matches_plain(results[True], folder, requests, dtype)


# Products with 17 to 64 rows and many rows of W run in a kernel of their own (activation rows
# shared through LDS): hidden size and feed-forward width are multiples of 512 here, and gate/up
# and the output head have 8192 rows, so a decode step of 40 requests takes it where a step of 8
# takes the kernel for few rows.  With more than 16 rows in_proj and qkv are also split over
# their input dimension (1024: two ranges) and the conv step and the qk-norm kernel add the
# partial sums.
MANY = {
    "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2",
    "hidden_size": 1024, "num_hidden_layers": 2, "layer_types": ["conv", "full_attention"],
    "num_attention_heads": 16, "num_key_value_heads": 4, "head_dim": 64,
    "intermediate_size": 4096, "block_auto_adjust_ff_dim": False,
    "vocab_size": 8192, "norm_eps": 1e-5, "rope_theta": 10000.0,
    "conv_L_cache": 3, "conv_bias": False, "tie_embedding": True,
    "max_position_embeddings": 512,
}


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_decode_steps_of_forty_requests(tmp_path, dtype):
    """Forty requests decoded side by side (and the same requests eight at a time) give the
    logits of each request alone in the plain implementation: the result does not depend on
    which product kernel the number of rows selects."""
    import copy
    from kappai_amd.cache import CacheManager
    from kappai_amd.config import config_from_dict
    from kappai_amd.engine import StepEntry, StepRunner
    from kappai_amd.weights import write_random_model
    folder = write_random_model(tmp_path / "many", config_from_dict(copy.deepcopy(MANY)), seed=6,
                                std=0.03, norm_jitter=0.05)
    n_req, n_decode = 40, 5
    lengths = [3 + (7 * i) % 23 + n_decode for i in range(n_req)]
    requests = make_requests(MANY["vocab_size"], lengths, seed=16)
    model = gpu_model(folder, dtype)
    ids = list(requests)
    for group in (40, 8):
        cache = CacheManager(model.cache_specs(), 16, n_req * 4, n_req)
        cache.allocate_storage(model.dtype, "cuda:0", poison=True)
        runner = StepRunner(model, cache, "cuda:0")
        got = {}
        for g0 in range(0, n_req, group):
            part = ids[g0:g0 + group]
            caches = {rid: cache.open(rid) for rid in part}
            # the prompts of the group in one step, then its decode steps
            entries = [StepEntry(caches[rid], requests[rid][:-n_decode],
                                 [len(requests[rid]) - n_decode - 1]) for rid in part]
            rows = runner.step(entries).cpu().numpy()
            for rid, row in zip(part, rows):
                got[(rid, len(requests[rid]) - n_decode - 1)] = row
            for s in range(n_decode):
                entries = [StepEntry(caches[rid], [requests[rid][s - n_decode]], [0])
                           for rid in part]
                rows = runner.step(entries).cpu().numpy()
                for rid, row in zip(part, rows):
                    got[(rid, len(requests[rid]) - n_decode + s)] = row
            for rid in part:
                cache.close(caches[rid])
        cache.check()
        from kappai_amd.kernels import ops
        assert ops.split_k_for(40, 3 * MANY["hidden_size"], MANY["hidden_size"]) > 1
        assert len(got) == n_req * (n_decode + 1)
        assert_matches_plain(got, folder, requests, dtype, what=f"{group} side by side")


MIXED_LENGTHS_MODEL = {
    "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2",
    "hidden_size": 512, "num_hidden_layers": 3,
    "layer_types": ["full_attention", "conv", "full_attention"],
    "num_attention_heads": 16, "num_key_value_heads": 8, "head_dim": 64,
    "intermediate_size": 1024, "block_auto_adjust_ff_dim": False,
    "vocab_size": 777, "norm_eps": 1e-5, "rope_theta": 10000.0,
    "conv_L_cache": 3, "conv_bias": False, "tie_embedding": True,
    "max_position_embeddings": 4096,
}


def test_requests_of_mixed_lengths_decoded_side_by_side(tmp_path):
    """Twelve requests of 150 to 2,300 tokens decoded side by side from captured graphs, in
    bfloat16: with eight kv heads the decode attention has more blocks than waves to aim at and
    settles the keys per split from the rows' own lengths, which change from request to request.
    Every decoded position against the plain implementation, and the graph's steps against the
    same steps run eagerly (bit for bit)."""
    import copy
    from kappai_amd.cache import CacheManager
    from kappai_amd.config import config_from_dict
    from kappai_amd.engine import StepEntry, StepRunner
    from kappai_amd.weights import write_random_model
    cfg = copy.deepcopy(MIXED_LENGTHS_MODEL)
    folder = write_random_model(tmp_path / "mixed", config_from_dict(cfg), seed=4, std=0.04,
                                norm_jitter=0.05)
    n_decode = 5
    lengths = [2300, 150, 1900, 640, 333, 2047, 1025, 512, 1500, 200, 897, 1211]
    requests = make_requests(cfg["vocab_size"], lengths, seed=31)
    model = gpu_model(folder, "bfloat16")
    ids = list(requests)
    results = {}
    for graphs in (True, False):
        cache = CacheManager(model.cache_specs(), 16, sum((n + 15) // 16 + 1 for n in lengths),
                             len(ids))
        cache.allocate_storage(model.dtype, "cuda:0", poison=True)
        runner = StepRunner(model, cache, "cuda:0", decode_graphs=graphs)
        caches = {rid: cache.open(rid) for rid in ids}
        got = {}
        for rid in ids:              # the prompts one by one, then the decode steps of all
            runner.step([StepEntry(caches[rid], requests[rid][:-n_decode], [])])
        for s in range(n_decode):
            entries = [StepEntry(caches[rid], [requests[rid][s - n_decode]], [0]) for rid in ids]
            rows = runner.step(entries).cpu().numpy()
            for rid, row in zip(ids, rows):
                got[(rid, len(requests[rid]) - n_decode + s)] = row
        for rid in ids:
            cache.close(caches[rid])
        cache.check()
        if graphs:
            assert runner.graph_replays >= n_decode - 2
        results[graphs] = got
    assert all(np.array_equal(results[True][k], results[False][k]) for k in results[True])
    assert_matches_plain(results[True], folder, requests, "bfloat16", what="mixed lengths")


# LFM2-1.2B as the benchmark runs it, all sixteen layers (attention at 2, 5, 8, 10, 12, 14): width
# 2048, 32 query heads over 8 kv heads of size 64, feed-forward 8192 from intermediate_size 12288,
# 65,536 tokens, tied head.  The plain implementation in float64 takes some ten seconds for the
# five requests; every schedule family replays the same five.
SIZES_1_2B = {
    "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2", "hidden_size": 2048,
    "num_hidden_layers": 16,
    "layer_types": ["full_attention" if i in (2, 5, 8, 10, 12, 14) else "conv" for i in range(16)],
    "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 64,
    "intermediate_size": 12288, "block_auto_adjust_ff_dim": True, "block_multiple_of": 256,
    "block_ffn_dim_multiplier": 1.0, "vocab_size": 65536, "norm_eps": 1e-5,
    "rope_theta": 1000000.0, "conv_L_cache": 3, "conv_bias": False, "tie_embedding": True,
    "max_position_embeddings": 128000,
}
LENGTHS_1_2B = [150, 97, 64, 80, 45]


@pytest.fixture(scope="module")
def sizes_1_2b_dir(tmp_path_factory):
    import copy
    from kappai_amd.config import config_from_dict
    from kappai_amd.weights import write_random_model
    cfg = config_from_dict(copy.deepcopy(SIZES_1_2B))
    assert cfg.ff_dim == 8192 and cfg.attention_layers == [2, 5, 8, 10, 12, 14]
    return write_random_model(tmp_path_factory.mktemp("sizes") / "m", cfg, seed=8, std=0.02,
                              norm_jitter=0.05)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_whole_1_2b_model(tmp_path, sizes_1_2b_dir, dtype):
    """The four schedule families at the size of LFM2-1.2B, every logit of every position: each
    request alone and whole; all but the last 32 tokens in one step, then one by one; portions of
    changing size; and mixed, three requests live at a time in a pool smaller than the five
    requests together, so that pages are used again."""
    folder = sizes_1_2b_dir
    requests = make_requests(SIZES_1_2B["vocab_size"], LENGTHS_1_2B, seed=17)
    total = sum(LENGTHS_1_2B)
    for family in ("whole", "prefill_then_decode", "changing_portions", "mixed"):
        kw = {"max_live": 3} if family == "mixed" else {}
        steps, index, peak = getattr(schedules, family)(requests, **kw)
        if family == "mixed":
            assert peak < total, "the pool must be reused"
        got = replay_in_process(folder, dtype, steps, index, peak, tmp_path / family)
        assert len(got) == total
        assert_matches_plain(got, folder, requests, dtype, what=family)
    _models.pop((str(folder), dtype), None)        # 2.3 GB on the GPU in bfloat16, 4.7 GB in float32


# A pool of more than 2^31 elements (8.7 GB of bfloat16 keys and as much of values in the one
# attention layer): the request's pages are the last of the pool, so every address of the
# store, prefill and decode kernels that does not fit 32 bits is used.
BIG_POOL = {
    "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2",
    "hidden_size": 128, "num_hidden_layers": 2, "layer_types": ["full_attention", "conv"],
    "num_attention_heads": 8, "num_key_value_heads": 8, "head_dim": 64,
    "intermediate_size": 256, "block_auto_adjust_ff_dim": False,
    "vocab_size": 300, "norm_eps": 1e-5, "rope_theta": 10000.0,
    "conv_L_cache": 3, "conv_bias": False, "tie_embedding": True,
    "max_position_embeddings": 1024,
}


@pytest.mark.parametrize("dtype", ["bfloat16"])
def test_pages_beyond_two_giga_elements(tmp_path, dtype):
    import copy
    from kappai_amd.cache import CacheManager
    from kappai_amd.config import config_from_dict
    from kappai_amd.engine.replay import TraceReplayer
    from kappai_amd.engine.step import StepRunner
    from kappai_amd.models import load_model
    from kappai_amd.weights import write_random_model
    folder = write_random_model(tmp_path / "m", config_from_dict(copy.deepcopy(BIG_POOL)), seed=9,
                                std=0.05, norm_jitter=0.05)
    model = load_model(folder, dtype, "cuda:0")
    page = 16
    per_page = 8 * page * 64
    pages = 2 * (2 ** 31 // per_page) + 40               # 4.3 G elements a pool
    cache = CacheManager(model.cache_specs(), page, pages, 4)
    cache.allocate_storage(model.dtype, "cuda:0")
    filler = cache.open("filler")                        # holds all pages but the last 24
    cache.extend(filler, (pages - 24) * page)
    requests = make_requests(BIG_POOL["vocab_size"], [150, 60], seed=19)
    plans = {"r0": (0, [100, 18] + [1] * 32), "r1": (1, [33, 27])}
    steps, index, peak = schedules.build(requests, plans)
    rep = TraceReplayer(StepRunner(model, cache, "cuda:0"), tmp_path / "out")
    outputs = {}
    for obj in steps:
        live = list(rep.live.values())
        res = rep.run_step(obj)
        assert all(min(b) >= pages - 24 for rc in live for b in rc.blocks if b)
        if res is not None:
            outputs[obj["step"]] = res
    cache.close(filler)
    cache.check()
    got = collect(index, outputs, model.vocab_size)
    assert_matches_plain(got, folder, requests, dtype)
    del rep, cache, model


def test_trace_semantics(tmp_path, model_dirs):
    """What a trace may do beside the regular schedules: places asked for out of order and
    twice, a request that is left out of steps and goes on later, a step that wants nothing
    (no file), a request ended by a step that brings no tokens for it, an empty step."""
    from kappai_amd.engine.replay import TraceReplayer, make_replay_cache
    from kappai_amd.engine.step import StepRunner
    cfg = TINY["C"][0]
    vocab = cfg["vocab_size"]
    requests = make_requests(vocab, [40, 23, 9], seed=18)
    a, b, c = requests["r0"], requests["r1"], requests["r2"]
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:10], "want": [9, 0, 9, 3]}], "end": []},
        {"step": 1, "entries": [{"id": "b", "tokens": b[:20], "want": []}], "end": []},
        {"step": 2, "entries": [{"id": "a", "tokens": a[10:12], "want": [1]},
                                {"id": "c", "tokens": c, "want": [8]}], "end": ["c"]},
        {"step": 3, "entries": [], "end": []},
        {"step": 4, "entries": [{"id": "b", "tokens": b[20:], "want": [2, 1, 0]}], "end": []},
        {"step": 5, "entries": [{"id": "a", "tokens": a[12:], "want": [27]}], "end": ["b"]},
        {"step": 6, "entries": [], "end": ["a"]},
    ]
    wanted = {0: [("r0", 9), ("r0", 0), ("r0", 9), ("r0", 3)], 2: [("r0", 11), ("r2", 8)],
              4: [("r1", 22), ("r1", 21), ("r1", 20)], 5: [("r0", 39)]}
    ref = plain_logits(model_dirs["C"], requests)
    scale = max(float(np.abs(v).max()) for v in ref.values())
    for dtype in ("float32", "bfloat16"):
        model = gpu_model(model_dirs["C"], dtype)
        cache = make_replay_cache(model, 64 + 64 + 64)
        cache.allocate_storage(model.dtype, "cuda:0", poison=True)
        out_dir = tmp_path / dtype
        rep = TraceReplayer(StepRunner(model, cache, "cuda:0"), out_dir)
        tol = tolerance(model_dirs["C"], requests, dtype)
        for obj in steps:
            res = rep.run_step(obj)
            if obj["step"] in wanted:
                rows = np.fromfile(out_dir / f"{obj['step']}.f32", dtype="<f4").reshape(-1, vocab)
                assert rows.shape[0] == len(wanted[obj["step"]]) and np.array_equal(rows, res)
                for row, (rid, pos) in zip(rows, wanted[obj["step"]]):
                    assert float(np.abs(row - ref[rid][pos]).max()) / scale < tol, (dtype, obj["step"], rid, pos)
            else:
                assert res is None and not (out_dir / f"{obj['step']}.f32").exists()
        cache.check()
        assert not cache.live_requests()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_the_order_of_the_entries_only_orders_the_logits(tmp_path, model_dirs, name, dtype):
    """A mixed step (two prompt portions, two single decoded tokens) in two different orders of
    its entries: the logits of every (request, place) are the same, only their order in the
    output follows the entries; so are the logits of the steps that come after, from the cache
    that the step left (kappai: a batch's segments are independent of each other,
    src/recipe/exec.c:704-758)."""
    from kappai_amd.engine.replay import TraceReplayer, make_replay_cache
    from kappai_amd.engine.step import StepRunner
    vocab = TINY[name][0]["vocab_size"]
    requests = make_requests(vocab, [40, 23, 31, 12], seed=19)
    a, b, c, d = (requests[f"r{i}"] for i in range(4))
    ids = {"a": "r0", "b": "r1", "c": "r2", "d": "r3"}
    before = [{"step": 0, "entries": [{"id": "a", "tokens": a[:17], "want": []},
                                      {"id": "b", "tokens": b[:22], "want": []}], "end": []},
              {"step": 1, "entries": [{"id": "c", "tokens": c[:9], "want": []}], "end": []}]
    mixed = [{"id": "a", "tokens": a[17:38], "want": [0, 20]}, {"id": "b", "tokens": b[22:23], "want": [0]},
             {"id": "c", "tokens": c[9:10], "want": [0]}, {"id": "d", "tokens": d, "want": [3, 11]}]
    first_place = {"a": 17, "b": 22, "c": 9, "d": 0}
    after = [{"step": 3, "entries": [{"id": "a", "tokens": a[38:], "want": [0, 1]},
                                     {"id": "c", "tokens": c[10:], "want": [20]}],
              "end": ["a", "b", "c", "d"]}]
    model = gpu_model(model_dirs[name], dtype)
    results = []
    for order in ([0, 1, 2, 3], [3, 2, 0, 1], [1, 3, 2, 0]):
        cache = make_replay_cache(model, 4 * 64)
        cache.allocate_storage(model.dtype, "cuda:0", poison=True)
        rep = TraceReplayer(StepRunner(model, cache, "cuda:0"), tmp_path / f"{dtype}{order[0]}")
        for obj in before:
            assert rep.run_step(obj) is None
        entries = [mixed[i] for i in order]
        rows = rep.run_step({"step": 2, "entries": entries, "end": []})
        got = {}
        at = 0
        for e in entries:
            for wnt in e["want"]:
                got[(ids[e["id"]], first_place[e["id"]] + wnt)] = rows[at]
                at += 1
        assert at == rows.shape[0] == 6
        later = rep.run_step(after[0])
        got[("r0", 38)], got[("r0", 39)], got[("r2", 30)] = later[0], later[1], later[2]
        cache.check()
        assert not cache.live_requests()
        results.append(got)
    # every order against the plain implementation, and the orders against each other
    assert_matches_plain(results[0], model_dirs[name], requests, dtype)
    for other in results[1:]:
        assert other.keys() == results[0].keys()
        for key in other:
            assert np.array_equal(other[key], results[0][key]), (key, "depends on the entries' order")
