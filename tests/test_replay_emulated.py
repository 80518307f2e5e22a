"""The engine's own logic (row tables, cache manager, step function, replay) against the
plain implementation, with the kernels replaced by torch CPU stand-ins.  No GPU needed.
The same schedules run on the GPU in test_replay_gpu.py."""
import pytest

import emulated_ops
import schedules
from replay_common import collect, first_bad, make_requests, plain_logits, worst_error
from tiny import TINY, write_tiny

from kappai_amd.engine.replay import TraceReplayer, make_replay_cache
from kappai_amd.models import load_model

FP32_TOL = 2e-5       # of the largest |logit|; float32 arithmetic against float64

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


def run_emulated(monkeypatch, model_dir, dtype, steps, index, max_tokens, tmp_path, page_size=16):
    emulated_ops.install(monkeypatch)
    model = load_model(model_dir, dtype, device="cpu")
    cache = make_replay_cache(model, max_tokens, page_size)
    cache.allocate_storage(model.dtype, "cpu", poison=True)
    rep = TraceReplayer(emulated_ops.make_cpu_runner(model, cache), tmp_path / "out")
    outputs = {}
    for obj in steps:
        res = rep.run_step(obj)
        if res is not None:
            outputs[obj["step"]] = res
        cache.check()
    assert not cache.live_requests()
    assert all(g.allocator.num_used == 0 for g in cache.paged_groups)
    return collect(index, outputs, model.vocab_size)


@pytest.mark.parametrize("name,family", [(n, f) for n in "ABC" for f in
                                         ("whole", "prefill_then_decode", "changing_portions", "mixed")]
                         + [(n, "mixed") for n in "DEFGH"])
def test_schedules_float32(monkeypatch, tmp_path, model_dirs, name, family):
    cfg = TINY[name][0]
    lengths = MIXED_LENGTHS[name] if family == "mixed" else LENGTHS[name]
    requests = make_requests(cfg["vocab_size"], lengths, seed=10)
    steps, index, peak = getattr(schedules, family)(requests)
    if family == "mixed":
        assert sum(len(t) for t in requests.values()) > peak, "the pool must be reused"
    got = run_emulated(monkeypatch, model_dirs[name], "float32", steps, index, peak, tmp_path)
    ref = plain_logits(model_dirs[name], requests)
    assert len(got) == sum(len(t) for t in requests.values())
    err, where = worst_error(got, ref)
    assert err < FP32_TOL, (err, where, first_bad(got, ref, FP32_TOL))


def test_a_step_without_entries_is_refused(monkeypatch, model_dirs):
    emulated_ops.install(monkeypatch)
    model = load_model(model_dirs["A"], "float32", device="cpu")
    cache = make_replay_cache(model, 64)
    runner = emulated_ops.make_cpu_runner(model, cache)
    runner.decode_graphs = True          # the path that used to look at the entries first
    with pytest.raises(ValueError, match="at least one entry"):
        runner.step([])
