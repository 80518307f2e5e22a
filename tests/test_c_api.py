"""The engine behind its C API (``csrc/engine_api.h``): called through ctypes from this process
(whose interpreter the library then uses) and from a C program of its own that is no Python
program (the library starts an interpreter).  Tokens, logits and numbers must be those of the
Python engine."""
import ctypes
import subprocess
from ctypes import POINTER, Structure, c_char_p, c_double, c_float, c_int, c_size_t, c_uint64, c_void_p
from pathlib import Path

import numpy as np
import pytest

from tiny import write_tiny

ROOT = Path(__file__).resolve().parent.parent
MAIN_SOURCE = Path(__file__).resolve().parent / "toy_parts" / "capi_main.c"
PROMPT_A = [3, 200, 17, 17, 0, 255, 9]
PROMPT_B = [41, 41, 100, 7, 8, 9, 250, 1, 2, 3, 4, 5]


class Config(Structure):
    _fields_ = [("model", c_char_p), ("dtype", c_char_p), ("device", c_int), ("ctx_size", c_int),
                ("page_size", c_int), ("num_pages", c_int), ("max_batch", c_int),
                ("token_budget", c_int), ("chunk", c_int), ("decode_graphs", c_int)]


class Sampling(Structure):
    _fields_ = [("temperature", c_float), ("top_k", c_int), ("top_p", c_float), ("min_p", c_float),
                ("repeat_penalty", c_float), ("repeat_last_n", c_int), ("seed", c_uint64),
                ("n_predict", c_int)]


class StepOutput(Structure):
    _fields_ = [("request_id", c_int), ("token", c_int), ("finished", c_int), ("reason", c_int)]


class Stats(Structure):
    _fields_ = [(n, c_double) for n in
                ("steps", "prompt_tokens", "prompt_seconds", "decoded_tokens", "decode_seconds",
                 "first_token_ms", "graph_replays", "preemptions", "free_pages", "vocab_size",
                 "ctx_size")]


def api():
    from kappai_amd.kernels.lib import library
    lib = library("engine_api")
    lib.kappai_engine_create.restype = c_void_p
    lib.kappai_engine_create.argtypes = [POINTER(Config)]
    lib.kappai_engine_destroy.argtypes = [c_void_p]
    lib.kappai_engine_error.restype = c_char_p
    lib.kappai_engine_add_request.argtypes = [c_void_p, POINTER(c_int), c_int, POINTER(Sampling)]
    lib.kappai_engine_step.argtypes = [c_void_p, POINTER(StepOutput), c_int]
    lib.kappai_engine_has_work.argtypes = [c_void_p]
    lib.kappai_engine_output.argtypes = [c_void_p, c_int, POINTER(c_int), c_int]
    lib.kappai_engine_release.argtypes = [c_void_p, c_int]
    lib.kappai_engine_abort.argtypes = [c_void_p, c_int]
    lib.kappai_engine_generate.argtypes = [c_void_p, POINTER(c_int), c_int, POINTER(Sampling),
                                           POINTER(c_int), c_int]
    lib.kappai_engine_get_stats.argtypes = [c_void_p, POINTER(Stats)]
    return lib


def test_defaults_and_refusals_without_a_gpu(tmp_path):
    """What needs no GPU: the defaults are kappai's (src/config.c:156-172), a configuration
    without a model is refused, and so is a model folder that does not exist or (here, where no
    GPU is visible) an engine without a GPU: null and a message, never a crash."""
    lib = api()
    s = Sampling()
    lib.kappai_sampling_default(ctypes.byref(s))
    assert (round(s.temperature, 2), s.top_k, round(s.top_p, 2), round(s.min_p, 2),
            s.repeat_penalty, s.repeat_last_n, s.seed, s.n_predict) == (0.8, 40, 0.9, 0.1, 1.0,
                                                                        64, 0, -1)
    lib.kappai_sampling_greedy(ctypes.byref(s), 5)
    assert (s.temperature, s.top_k, s.top_p, s.min_p, s.n_predict) == (0.0, 0, 1.0, 0.0, 5)
    c = Config()
    lib.kappai_engine_config_default(ctypes.byref(c))
    assert lib.kappai_engine_create(ctypes.byref(c)) is None
    assert b"no model folder" in lib.kappai_engine_error()
    c.model = str(tmp_path / "nowhere").encode()
    assert lib.kappai_engine_create(ctypes.byref(c)) is None
    assert lib.kappai_engine_error()                   # (which of the two reasons depends on the box)
    assert lib.kappai_engine_step(None, None, 0) == -1
    assert b"no engine" in lib.kappai_engine_error()
    lib.kappai_engine_destroy(None)


def python_engine_tokens(folder, dtype, n_predict):
    from kappai_amd.engine import Engine
    from kappai_amd.sampling import SamplingParams
    eng = Engine(str(folder), dtype=dtype, num_pages=64, max_batch=4)
    both = eng.generate([PROMPT_A, PROMPT_B], SamplingParams.greedy(n_predict=n_predict))
    (alone,) = eng.generate([PROMPT_A], SamplingParams.greedy(n_predict=n_predict))
    eng.shutdown()
    return both, alone


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_c_api_through_ctypes(tmp_path, dtype):
    """Requests added, stepped and read through the C functions give the Python engine's tokens;
    an abort ends a request; the numbers add up."""
    folder = write_tiny("A", tmp_path / "a")
    want_both, want_alone = python_engine_tokens(folder, dtype, 6)
    lib = api()
    c = Config()
    lib.kappai_engine_config_default(ctypes.byref(c))
    c.model, c.dtype, c.num_pages, c.max_batch = str(folder).encode(), dtype.encode(), 64, 4
    engine = lib.kappai_engine_create(ctypes.byref(c))
    assert engine, lib.kappai_engine_error()
    greedy = Sampling()
    lib.kappai_sampling_greedy(ctypes.byref(greedy), 6)
    ids = []
    for prompt in (PROMPT_A, PROMPT_B):
        arr = (c_int * len(prompt))(*prompt)
        ids.append(lib.kappai_engine_add_request(engine, arr, len(prompt), ctypes.byref(greedy)))
    assert ids == [0, 1], lib.kappai_engine_error()
    seen = {0: [], 1: []}
    out = (StepOutput * 1)()                     # one place only: the rest waits for the next call
    while lib.kappai_engine_has_work(engine) == 1:
        n = lib.kappai_engine_step(engine, out, 1)
        assert n >= 0, lib.kappai_engine_error()
        for o in out[:n]:
            if o.token >= 0:
                seen[o.request_id].append(o.token)
            assert o.finished in (0, 1) and (o.reason == 2) == bool(o.finished)
    assert [seen[0], seen[1]] == want_both
    buf = (c_int * 3)()
    assert lib.kappai_engine_output(engine, 1, buf, 3) == 6 and list(buf) == want_both[1][:3]
    assert lib.kappai_engine_release(engine, 1) == 1 and lib.kappai_engine_release(engine, 1) == 0
    assert lib.kappai_engine_output(engine, 1, buf, 3) == -1
    assert b"no request 1" in lib.kappai_engine_error()
    # the blocking call, and a request that is stopped
    tokens = (c_int * 16)()
    arr = (c_int * len(PROMPT_A))(*PROMPT_A)
    assert lib.kappai_engine_generate(engine, arr, len(PROMPT_A), ctypes.byref(greedy), tokens,
                                      16) == 6
    assert list(tokens[:6]) == want_alone
    rid = lib.kappai_engine_add_request(engine, arr, len(PROMPT_A), ctypes.byref(greedy))
    assert lib.kappai_engine_step(engine, out, 1) >= 0
    assert lib.kappai_engine_abort(engine, rid) == 1 and lib.kappai_engine_abort(engine, rid) == 0
    bad = (c_int * 2)(5, 100000)
    assert lib.kappai_engine_add_request(engine, bad, 2, ctypes.byref(greedy)) == -1
    assert b"outside the vocabulary" in lib.kappai_engine_error()
    stats = Stats()
    assert lib.kappai_engine_get_stats(engine, ctypes.byref(stats)) == 0
    assert stats.vocab_size == 256 and stats.decoded_tokens >= 15 and stats.free_pages == 64
    lib.kappai_engine_destroy(engine)


@pytest.mark.gpu
def test_c_api_from_a_c_program(tmp_path):
    """A C program that loads the library and has no interpreter of its own: the same tokens as
    the Python engine, the raw step function's logits point at the tokens that the plain
    implementation's logits point at, a refused call says why."""
    from kappai_amd.kernels.lib import _find_built, _source_hash
    from plain import lfm2 as plain
    folder = write_tiny("A", tmp_path / "a")
    want_both, want_alone = python_engine_tokens(folder, "float32", 5)
    exe = tmp_path / "capi_main"
    subprocess.run(["gcc", "-O1", "-I", str(ROOT / "kappai_amd" / "csrc"), str(MAIN_SOURCE), "-o",
                    str(exe), "-ldl"], check=True)
    so = _find_built("engine_api", _source_hash("engine_api"))
    assert so is not None, "the library is built before the GPU tests run"
    proc = subprocess.run([str(exe), str(so), str(folder), "float32", "5"], capture_output=True,
                          text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr
    lines = dict(line.split(":", 1) if ":" in line else (line, "") for line in
                 proc.stdout.strip().splitlines())
    assert [int(t) for t in lines["request 0"].split()] == want_both[0]
    assert [int(t) for t in lines["request 1"].split()] == want_both[1]
    assert [int(t) for t in lines["generate"].split()] == want_alone
    assert "reported 10 ended 2" in proc.stdout
    cfg, w = plain.read_model_dir(folder)
    b = plain.forward(cfg, w, PROMPT_B[:7])
    a = plain.forward(cfg, w, PROMPT_A[:3])
    assert f"forward argmax {int(b[4].argmax())}" in proc.stdout
    for r, row in enumerate((b[5], b[6], a[2])):
        assert f"forward row {r} argmax {int(row.argmax())}" in proc.stdout
    assert "refused -1" in proc.stdout and "do not fit 10 floats" in proc.stdout
    assert "vocab 256" in proc.stdout
