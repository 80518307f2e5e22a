"""Generation through the Python entry point and the command line, against the plain
implementation: greedy chains, sampled chains from a fixed seed, prompts cut into portions
and mixed with decoding, and preemption when pages run out."""
import json
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest

from plain import lfm2 as P
from plain import sampler as S
from tiny import TINY, write_tiny

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parent.parent


@pytest.fixture(scope="module")
def model_dirs(tmp_path_factory):
    base = tmp_path_factory.mktemp("models")
    return {name: write_tiny(name, base / name) for name in TINY}


def prompts_for(name, lengths, seed):
    rng = np.random.default_rng(seed)
    return [[int(t) for t in rng.integers(0, TINY[name][0]["vocab_size"], size=n)] for n in lengths]


def plain_generate(model_dir, prompt, n, make_sampler):
    """Token by token with the plain implementation: the whole sequence again for every
    token, no cache."""
    cfg, w = P.read_model_dir(model_dir)
    sampler = make_sampler()
    for t in prompt:
        sampler.observe(t)
    toks, out, rows = list(prompt), [], []
    for _ in range(n):
        logits = P.forward(cfg, w, toks)[-1]
        tok = sampler.sample(logits.astype(np.float32))
        sampler.observe(tok)
        rows.append(logits)
        toks.append(tok)
        out.append(tok)
    return out, rows


def test_greedy_float32_tiny_a(model_dirs):
    """Two prompts of 7 and 12 ids, then 8 greedy tokens each."""
    from kappai_amd.engine import Engine
    from kappai_amd.sampling import SamplingParams
    prompts = prompts_for("A", [7, 12], seed=0)
    eng = Engine(str(model_dirs["A"]), dtype="float32", num_pages=64, max_batch=4)
    got = eng.generate(prompts, SamplingParams.greedy(n_predict=8))
    for p, g in zip(prompts, got):
        want, _ = plain_generate(model_dirs["A"], p, 8, lambda: S.PlainSampler(1, temperature=0.0))
        assert g == want
    assert eng.cache.num_free_pages() == 64 and eng.cache.num_free_slots == 4
    assert eng.metrics.decode_tokens == 14 and eng.metrics.prefill_tokens == 19
    assert eng.metrics.line("pp,tg,ttft").startswith("[ PP: ")


def test_sampled_float32_tiny_b_in_portions(model_dirs):
    """Three prompts of 5, 17 and 33 ids, prefilled in portions of 4 beside decoding, then 10
    tokens each at temperature 0.8 from a fixed seed (whole-vocabulary draw)."""
    from kappai_amd.engine import Engine
    from kappai_amd.sampling import SamplingParams
    prompts = prompts_for("B", [5, 17, 33], seed=1)
    params = SamplingParams(temperature=0.8, top_k=0, top_p=1.0, min_p=0.0, seed=1234, n_predict=10)
    eng = Engine(str(model_dirs["B"]), dtype="float32", num_pages=64, max_batch=4, chunk=4,
                 token_budget=9)
    got = eng.generate(prompts, params)
    assert eng.metrics.steps > 10
    for i, (p, g) in enumerate(zip(prompts, got)):
        want, _ = plain_generate(model_dirs["B"], p, 10, lambda: S.PlainSampler(
            1234 + i, temperature=0.8, top_k=0, top_p=1.0, min_p=0.0))
        assert g == want, (i, g, want)


def test_every_way_of_drawing_in_one_batch():
    """One batch of rows that each draw differently (greedy, the whole vocabulary, narrowed to a
    few, a top-k above what the kernel for narrowed rows holds, a repeat penalty) over several
    steps, every row against a plain sampler of its own with the same seed: a row's tokens do not
    depend on what its neighbours ask for."""
    import torch
    from kappai_amd.sampling import RequestSampler, Sampler, SamplingParams
    V = 3001
    opts = [dict(temperature=0.0), dict(temperature=0.9, top_k=0, top_p=1.0, min_p=0.0),
            dict(temperature=0.8, top_k=40, top_p=0.9, min_p=0.1),
            dict(temperature=1.5, top_k=2000, top_p=0.98, min_p=0.0),
            dict(temperature=1.1, top_k=1500, top_p=1.0, min_p=0.001),
            dict(temperature=0.7, top_k=12, top_p=1.0, min_p=0.0, repeat_penalty=1.3, repeat_last_n=4),
            dict(temperature=2.0, top_k=3000, top_p=1.0, min_p=0.0)]
    ours = [RequestSampler(SamplingParams(seed=11 + i, **o)) for i, o in enumerate(opts)]
    plain = [S.PlainSampler(11 + i, **{"top_k": 40, "top_p": 0.9, "min_p": 0.1, **o})
             for i, o in enumerate(opts)]
    sampler = Sampler()
    rng = np.random.default_rng(8)
    for step in range(6):
        logits = (rng.normal(size=(len(opts), V)) * 2.5).astype(np.float32)
        got = sampler.sample(torch.from_numpy(logits).to("cuda:0"), ours)
        for i, tok in enumerate(got):
            want = plain[i].sample(logits[i].copy())
            assert tok == want, (step, i, opts[i], tok, want)
            ours[i].observe([tok])
            plain[i].observe(tok)


def test_default_options_and_repeat_penalty(model_dirs):
    """kappai's default options (top-k 40, top-p 0.9, min-p 0.1) and a repeat penalty."""
    from kappai_amd.engine import Engine
    from kappai_amd.sampling import SamplingParams
    prompts = prompts_for("C", [9, 21], seed=2)
    params = SamplingParams(seed=77, n_predict=12, repeat_penalty=1.3, repeat_last_n=8)
    eng = Engine(str(model_dirs["C"]), dtype="float32", num_pages=32, max_batch=2)
    got = eng.generate(prompts, params)
    for i, (p, g) in enumerate(zip(prompts, got)):
        want, _ = plain_generate(model_dirs["C"], p, 12, lambda: S.PlainSampler(
            77 + i, repeat_penalty=1.3, repeat_last_n=8))
        assert g == want, (i, g, want)


def test_repeat_penalty_goes_ahead_of_its_tokens(model_dirs):
    """Requests with a repeat penalty (windows of 8 and 64 tokens, one over the prompt's end)
    beside requests without: the steps are queued before the tokens of the steps before them
    have been read (the recent tokens are kept on the GPU), with so few pages that requests are
    preempted and computed again, and every request's tokens are those of the plain
    implementation with a plain sampler of the same seed, and those of a run in which every step
    is waited for."""
    from kappai_amd.engine import Engine, EngineConfig
    from kappai_amd.sampling import SamplingParams
    prompts = prompts_for("C", [9, 21, 14, 30, 5], seed=4)
    opts = [dict(repeat_penalty=1.3, repeat_last_n=8), dict(repeat_penalty=1.6, repeat_last_n=64),
            dict(), dict(repeat_penalty=1.15, repeat_last_n=3, temperature=0.0), dict()]
    params = [SamplingParams(seed=50, n_predict=20, **o) for o in opts]
    results = {}
    for pipeline in (True, False):
        eng = Engine(EngineConfig(model=str(model_dirs["C"]), dtype="float32", num_pages=14,
                                  page_size=8, max_batch=4, chunk=6, token_budget=12,
                                  pipeline=pipeline))
        results[pipeline] = eng.generate(prompts, params)
        if pipeline:
            assert eng.pipelined_steps > 0, "nothing was queued ahead"
            assert eng.scheduler.preempted_total > 0, "the pool was meant to be too small"
        eng.shutdown()
    assert results[True] == results[False]
    for i, (p, g) in enumerate(zip(prompts, results[True])):
        want, _ = plain_generate(model_dirs["C"], p, 20, lambda: S.PlainSampler(
            50 + i, **{"top_k": 40, "top_p": 0.9, "min_p": 0.1, **opts[i]}))
        assert g == want, (i, g, want)


def test_repeat_penalty_over_a_window_longer_than_the_ring(model_dirs):
    """A repeat penalty over the last 300 tokens (more than the 256 kept on the GPU) beside one
    over 8: such steps take the host's lists and are waited for, and when the long window's
    request has ended the other goes on from its ring, which is written anew; every request's
    tokens are the plain implementation's."""
    from kappai_amd.engine import Engine
    from kappai_amd.sampling import SamplingParams
    prompts = prompts_for("C", [310, 12], seed=6)
    opts = [dict(repeat_penalty=1.4, repeat_last_n=300, n_predict=6),
            dict(repeat_penalty=1.3, repeat_last_n=8, n_predict=24)]
    params = [SamplingParams(seed=60, **o) for o in opts]
    eng = Engine(str(model_dirs["C"]), dtype="float32", num_pages=64, max_batch=2)
    got = eng.generate(prompts, params)
    assert eng.pipelined_steps > 0, "the steps after the long window's end were meant to go ahead"
    for i, (p, g) in enumerate(zip(prompts, got)):
        o = dict(opts[i])
        n = o.pop("n_predict")
        want, _ = plain_generate(model_dirs["C"], p, n, lambda: S.PlainSampler(
            60 + i, **{"top_k": 40, "top_p": 0.9, "min_p": 0.1, **o}))
        assert g == want, (i, g, want)


def test_greedy_bfloat16_follows_the_plain_logits(model_dirs):
    """In bfloat16 the chain may leave the plain one at a near tie; every token the engine
    picks must be (nearly) the best under the plain logits for the engine's own prefix."""
    from kappai_amd.engine import Engine
    from kappai_amd.sampling import SamplingParams
    prompts = prompts_for("B", [11, 30], seed=3)
    eng = Engine(str(model_dirs["B"]), dtype="bfloat16", num_pages=64, max_batch=4, chunk=7)
    got = eng.generate(prompts, SamplingParams.greedy(n_predict=12))
    cfg, w = P.read_model_dir(model_dirs["B"])
    for p, g in zip(prompts, got):
        assert len(g) == 12
        logits = P.forward(cfg, w, p + g)
        for j, tok in enumerate(g):
            row = logits[len(p) - 1 + j]
            assert row[tok] >= row.max() - 0.03 * np.abs(row).max(), (j, tok, int(row.argmax()))


def test_greedy_bfloat16_in_queued_decode_runs_follows_the_plain_logits(model_dirs):
    """Three requests decoded 40 tokens each, mostly in runs of eight queued graph replays whose
    tokens stay on the GPU between steps (with dummy rows: three requests run in the graph for
    four): every token chosen is the best, or as good as the best within twice the error bound
    of a bfloat16 logit, under the plain logits of the engine's own prefix."""
    from replay_common import BF16_MAX_FACTOR, bf16_bounds
    from kappai_amd.engine import Engine
    from kappai_amd.sampling import SamplingParams
    prompts = prompts_for("B", [19, 6, 33], seed=8)
    eng = Engine(str(model_dirs["B"]), dtype="bfloat16", num_pages=64, max_batch=4, decode_run=8)
    got = eng.generate(prompts, SamplingParams.greedy(n_predict=40))
    assert eng.decode_runs >= 3 and eng.runner.graph_replays >= 24
    cfg, w = P.read_model_dir(model_dirs["B"])
    for i, (p, g) in enumerate(zip(prompts, got)):
        assert len(g) == 40
        seq = {f"s{i}": p + g}
        logits = P.forward(cfg, w, p + g)
        keys = [(f"s{i}", len(p) - 1 + j) for j in range(len(g))]
        bound = BF16_MAX_FACTOR * bf16_bounds(model_dirs["B"], seq, keys)[0] * np.abs(logits).max()
        for j, tok in enumerate(g):
            row = logits[len(p) - 1 + j]
            assert row[tok] >= row.max() - 2 * bound, (i, j, tok, int(row.argmax()), bound)


def test_preemption_gives_the_same_tokens(model_dirs):
    """With so few pages that requests are preempted and computed again, greedy output is what
    it is with plenty of pages."""
    from kappai_amd.engine import Engine
    from kappai_amd.sampling import SamplingParams
    prompts = prompts_for("A", [30, 25, 28, 9], seed=4)
    params = SamplingParams.greedy(n_predict=20)
    roomy = Engine(str(model_dirs["A"]), dtype="float32", num_pages=64, max_batch=4)
    want = roomy.generate(prompts, params)
    tight = Engine(str(model_dirs["A"]), dtype="float32", num_pages=8, page_size=16, max_batch=4,
                   token_budget=40)
    got = tight.generate(prompts, params)
    assert tight.scheduler.preempted_total > 0
    assert got == want
    assert tight.cache.num_free_pages() == 8
    too_long = Engine(str(model_dirs["A"]), dtype="float32", num_pages=2, max_batch=2)
    with pytest.raises(RuntimeError, match="context exceeds cache"):
        too_long.generate([list(range(40))], params)


def test_abort_leaves_the_others_alone(model_dirs):
    """One of three requests is aborted after a few steps (inside its decoding, while decode
    graphs and queued decode runs are in use): the others end with the tokens they have without
    it, its pages and slot are back, and a request added afterwards runs in what it freed."""
    from kappai_amd.engine import Engine
    from kappai_amd.sampling import SamplingParams
    prompts = prompts_for("B", [9, 21, 14], seed=6)
    params = SamplingParams.greedy(n_predict=24)
    alone = Engine(str(model_dirs["B"]), dtype="float32", num_pages=32, max_batch=3)
    want = alone.generate([prompts[0], prompts[2]], params)
    eng = Engine(str(model_dirs["B"]), dtype="float32", num_pages=32, max_batch=3)
    ids = [eng.add_request(p, params) for p in prompts]
    for _ in range(3):
        eng.step()
    victim = eng.requests[ids[1]]
    assert 0 < len(victim.output) < 24
    assert eng.abort(ids[1]) and not eng.abort(ids[1]) and not eng.abort("no such request")
    assert victim.finish_reason == "aborted" and eng.cache.num_free_slots == 1
    late = eng.add_request(prompts[1], params)
    while eng.has_unfinished():
        eng.step()
    assert [eng.requests[ids[0]].output, eng.requests[ids[2]].output] == want
    assert len(eng.requests[late].output) == 24
    assert eng.cache.num_free_pages() == 32 and eng.cache.num_free_slots == 3


def test_random_engine_options_give_the_same_tokens(model_dirs):
    """Thirty random combinations of page size, pool size (down to what the longest request
    needs plus a page), live requests, token budget, longest portion and queued decode steps,
    with greedy and seeded sampled requests: in float32 the tokens are those of a roomy engine
    that takes every step by itself, and every page and slot comes back."""
    import random
    from kappai_amd.engine import Engine
    from kappai_amd.sampling import SamplingParams
    rng = random.Random(7)
    for trial in range(30):
        name = rng.choice(["A", "B", "G", "H"])
        vocab = TINY[name][0]["vocab_size"]
        n_req = rng.randint(1, 7)
        prompts = [[rng.randrange(vocab) for _ in range(rng.randint(1, 60))] for _ in range(n_req)]
        params = [SamplingParams.greedy(n_predict=rng.randint(1, 30)) if rng.random() < 0.6 else
                  SamplingParams(temperature=0.8, top_k=rng.choice([0, 5, 40]),
                                 top_p=rng.choice([1.0, 0.9]), min_p=rng.choice([0.0, 0.1]),
                                 seed=rng.randint(1, 99), n_predict=rng.randint(1, 30))
                  for _ in range(n_req)]
        page = rng.choice([4, 16, 16, 32, 48, 64])
        longest = max(len(p) + sp.n_predict for p, sp in zip(prompts, params))
        least = (longest + page - 1) // page + 1
        options = dict(page_size=page, num_pages=rng.choice([least, least + 2, 4 * least, 64]),
                       max_batch=rng.choice([1, 2, 3, 8]),
                       token_budget=rng.choice([1, 3, 17, 64, 2048]),
                       chunk=rng.choice([1, 2, 5, 33, 2048]), decode_run=rng.choice([1, 2, 8]),
                       warm_kernels=rng.random() < 0.5, pipeline=rng.random() < 0.7)
        roomy = Engine(str(model_dirs[name]), dtype="float32", num_pages=256, page_size=16,
                       max_batch=8, decode_run=1, warm_kernels=False, pipeline=False)
        want = roomy.generate(prompts, params)
        eng = Engine(str(model_dirs[name]), dtype="float32", **options)
        got = eng.generate(prompts, params)
        assert got == want, (trial, name, options, [len(p) for p in prompts])
        assert eng.cache.num_free_slots == options["max_batch"]
        assert eng.cache.num_free_pages() == options["num_pages"]


def test_fragment_order_changes_no_token(tmp_path):
    """The matrices kept in fragment order, and the normalised rows of a decode step in that
    order, are layouts only: a model with and without them generates the same tokens in
    bfloat16, greedy and sampled, through prompt portions, decode graphs and queued decode steps
    (sizes at which every matrix can be kept so; the tied head's matrix is then the embedding's
    table as well)."""
    import copy
    from kappai_amd.config import config_from_dict
    from kappai_amd.engine import Engine
    from kappai_amd.kernels import tuning
    from kappai_amd.sampling import SamplingParams
    from kappai_amd.weights import write_random_model
    raw = {"architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2", "hidden_size": 256,
           "num_hidden_layers": 4,
           "layer_types": ["conv", "full_attention", "conv", "full_attention"],
           "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 64,
           "intermediate_size": 512, "block_auto_adjust_ff_dim": False, "vocab_size": 1024,
           "norm_eps": 1e-5, "rope_theta": 10000.0, "conv_L_cache": 3, "conv_bias": False,
           "tie_embedding": True, "max_position_embeddings": 1024}
    folder = write_random_model(tmp_path / "m", config_from_dict(copy.deepcopy(raw)), seed=11,
                                std=0.05, norm_jitter=0.05)
    rng = np.random.default_rng(12)
    prompts = [[int(t) for t in rng.integers(0, 1024, size=n)]
               for n in (40, 3, 75, 18, 9, 5, 31, 12, 22, 7)]
    params = [SamplingParams.greedy(n_predict=24), SamplingParams(seed=3, n_predict=24),
              SamplingParams.greedy(n_predict=10), SamplingParams(seed=4, top_k=0, n_predict=24),
              SamplingParams.greedy(n_predict=24)] * 2
    assert len(prompts) >= tuning.FRAGMENT_ROWS_MIN      # decode steps with rows enough for the order
    outs = []
    from kappai_amd.kernels import ops
    assert tuning.FRAGMENT_ORDER and tuning.FRAGMENT_ROWS
    try:
        for order, rows in ((True, True), (False, True), (True, False), (False, False)):
            tuning.FRAGMENT_ORDER, tuning.FRAGMENT_ROWS = order, rows
            eng = Engine(str(folder), dtype="bfloat16", num_pages=128, max_batch=10, chunk=32,
                         token_budget=48)
            kept = [blk.feed_forward.down.weight for blk in eng.model.layers]
            kept += [blk.mixer.out.weight if hasattr(blk.mixer, "out") else blk.mixer.in_proj.weight
                     for blk in eng.model.layers]
            kept += [eng.model.head.linear.weight, eng.model.embedding.table]
            assert all(isinstance(w, ops.InFragments) == order for w in kept)
            outs.append(eng.generate(prompts, params))
    finally:
        tuning.FRAGMENT_ORDER, tuning.FRAGMENT_ROWS = True, True
    assert outs[0] == outs[1] == outs[2] == outs[3]


def test_command_line(model_dirs, tmp_path):
    prompt = prompts_for("A", [7], seed=5)[0]
    want, _ = plain_generate(model_dirs["A"], prompt, 6, lambda: S.PlainSampler(1, temperature=0.0))
    out = subprocess.run(
        [sys.executable, "-m", "kappai_amd", "-m", str(model_dirs["A"]), "--dtype", "float32",
         "-p", ",".join(map(str, prompt)), "-n", "6", "-t", "0", "--metrics", "pp,tg,ttft",
         "--num-pages", "16", "--dump-logits", str(tmp_path / "lg.f32")],
        cwd=str(ROOT), capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr
    assert [int(t) for t in out.stdout.split()] == want
    assert "[ PP: " in out.stderr and "TG: " in out.stderr and "TTFT: " in out.stderr
    assert (tmp_path / "lg.f32").stat().st_size == 6 * 256 * 4
    # random-weights mode from a config.json
    cfgp = tmp_path / "cfg.json"
    cfgp.write_text(json.dumps(TINY["C"][0]))
    out = subprocess.run(
        [sys.executable, str(ROOT / "bin" / "kappai-cli"), "--random-weights", str(cfgp),
         "--weight-seed", "3", "-n", "4", "-s", "5", "--num-pages", "16", "1 2 3"],
        cwd=str(tmp_path), capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr
    assert len(out.stdout.split()) == 4
    # random-weights mode from the name of a shape, with the weights' spread given: the folder is
    # the one that the same call of the library writes (Tiny B: norm weights 1 + N(0, 0.1))
    made = tmp_path / "made"
    out = subprocess.run(
        [sys.executable, str(ROOT / "bin" / "kappai-cli"), "--random-weights", "tiny-b",
         "--model", str(made), "--weight-seed", "1", "--weight-std", "0.05", "--norm-jitter",
         "0.1", "--dtype", "float32", "-n", "5", "-t", "0", "--num-pages", "16", "7 8 9 10"],
        cwd=str(tmp_path), capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr
    same = write_tiny("B", tmp_path / "same")
    assert (made / "model.safetensors").read_bytes() == (same / "model.safetensors").read_bytes()
    want, _ = plain_generate(same, [7, 8, 9, 10], 5, lambda: S.PlainSampler(1, temperature=0.0))
    assert [int(t) for t in out.stdout.split()] == want
    out = subprocess.run(
        [sys.executable, str(ROOT / "bin" / "kappai-cli"), "--random-weights", "lfm2-9b", "1 2"],
        cwd=str(tmp_path), capture_output=True, text=True, timeout=300)
    assert out.returncode == 2 and "neither a file nor one of the shapes" in out.stderr


def test_command_line_times_by_stage(model_dirs):
    """--time: the tokens are those of a run without it, and after the run there is a table of
    the time by stage for the steps with prompt portions and one for the decode steps."""
    prompt = prompts_for("B", [21], seed=9)[0]
    base = [sys.executable, "-m", "kappai_amd", "-m", str(model_dirs["B"]), "--dtype", "bfloat16",
            "-p", ",".join(map(str, prompt)), "-n", "5", "-t", "0", "--num-pages", "16"]
    plain_run = subprocess.run(base, cwd=str(ROOT), capture_output=True, text=True, timeout=300)
    timed = subprocess.run(base + ["--time"], cwd=str(ROOT), capture_output=True, text=True,
                           timeout=300)
    assert timed.returncode == 0, timed.stderr
    assert timed.stdout.split() == plain_run.stdout.split()
    err = timed.stderr
    assert "[profile] prefill  accounted=" in err and "[profile] decode  accounted=" in err
    decode = err[err.index("[profile] decode"):]
    for stage in ("embd", "matmul_qkv", "matmul_attn_out", "matmul_in_proj", "matmul_ffn_gate_up",
                  "matmul_ffn_down", "rope_kvput", "attn", "logits_matmul", "sample"):
        assert f"  {stage} " in decode, (stage, decode)
    # 4 decode steps x 3 attention layers
    row = next(line for line in decode.splitlines() if line.startswith("  attn "))
    assert int(row.split()[2]) == 12, row


def test_smoke_entry():
    sys.path.insert(0, str(ROOT))
    import __graft_entry__
    __graft_entry__.smoke()


def _engine(model_dir, dtype, **kw):
    from kappai_amd.engine import Engine, EngineConfig
    return Engine(EngineConfig(model=str(model_dir), dtype=dtype, num_pages=256, max_batch=8, **kw))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_runs_give_the_same_tokens(model_dirs, dtype):
    """Several decode steps queued back to back (each step's token handed to the next on the
    GPU) must give exactly the tokens of steps that are waited for one by one: greedy and
    sampled requests side by side, ending at different lengths, inside and at the end of runs."""
    from kappai_amd.sampling import SamplingParams
    prompts = prompts_for("B", [9, 30, 4, 17, 11], seed=21)
    params = [SamplingParams.greedy(n_predict=41), SamplingParams.greedy(n_predict=23),
              SamplingParams(temperature=0.9, top_k=0, top_p=1.0, min_p=0.0, seed=5, n_predict=36),
              SamplingParams(temperature=0.7, top_k=12, top_p=0.9, min_p=0.05, seed=6, n_predict=29),
              SamplingParams.greedy(n_predict=2)]
    results = {}
    for run_len in (0, 1, 8, 3):         # 0: no captured graphs at all, every step eager
        eng = _engine(model_dirs["B"], dtype, decode_run=max(run_len, 1))
        if run_len == 0:
            eng.runner.decode_graphs = False
        results[run_len] = eng.generate(prompts, params)
        eng.cache.check()
        assert eng.cache.num_free_pages() == 256 and eng.cache.num_free_slots == 8
        if run_len > 1:
            assert eng.runner.graph_replays > 20
        assert (eng.runner.graph_replays == 0) == (run_len == 0)
        assert [len(o) for o in results[run_len]] == [41, 23, 36, 29, 2]
    # the batch shrinks from 5 to 1 as requests end: steps of 5 and 3 rows are replayed from the
    # graphs of 8 and 4 rows with dummy rows
    assert results[1] == results[0]
    assert results[8] == results[1]
    assert results[3] == results[1]


def test_end_of_sequence_inside_a_decode_run(model_dirs, tmp_path):
    """A request that draws its end-of-sequence token in the middle of a run ends there: the
    tokens of the steps that were queued behind it are dropped, its pages and its slot come
    back, and the other requests are not disturbed."""
    from kappai_amd.sampling import SamplingParams
    prompts = prompts_for("B", [6, 13, 8], seed=22)
    params = [SamplingParams(temperature=1.0, top_k=0, top_p=1.0, min_p=0.0, seed=40 + i,
                             n_predict=40) for i in range(3)]
    eng = _engine(model_dirs["B"], "float32", decode_run=1)
    free = eng.generate(prompts, params)
    # a token that request 0 draws late enough to fall inside a run, and that nobody drew before
    pick = None
    for k in range(12, 40):
        t = free[0][k]
        if t not in free[0][:k] and all(t not in o for o in free[1:]):
            pick = (k, t)
            break
    assert pick is not None, "the chains share all their tokens"
    k, eos = pick
    cfg = json.loads((model_dirs["B"] / "config.json").read_text())
    cfg["eos_token_id"] = eos
    folder = tmp_path / "with_eos"
    folder.mkdir()
    (folder / "config.json").write_text(json.dumps(cfg))
    (folder / "model.safetensors").write_bytes((model_dirs["B"] / "model.safetensors").read_bytes())
    for run_len in (1, 8):
        eng = _engine(folder, "float32", decode_run=run_len)
        got = eng.generate(prompts, params)
        assert got[0] == free[0][:k + 1] and got[0][-1] == eos
        assert got[1] == free[1] and got[2] == free[2]
        eng.cache.check()
        assert eng.cache.num_free_pages() == 256 and eng.cache.num_free_slots == 8


def test_steps_ahead_of_their_tokens_give_the_same_tokens(model_dirs, tmp_path):
    """Steps with prompt portions in them are queued before the tokens of the step before have
    been read: the requests that decode beside the prompts take their tokens on the GPU.  The
    tokens must be those of steps that are waited for one by one: greedy and sampled requests,
    one that draws its end-of-sequence token while prompts are under way (it has taken a step
    too many by the time that is known), a roomy pool and one so tight that the scheduler has
    to ask for the tokens before it preempts."""
    import random
    from kappai_amd.engine import Engine, EngineConfig
    from kappai_amd.sampling import SamplingParams
    rng = random.Random(5)
    vocab = TINY["B"][0]["vocab_size"]
    n = 14
    prompts = [[rng.randrange(vocab) for _ in range(rng.randint(3, 150))] for _ in range(n)]
    params = [SamplingParams.greedy(n_predict=rng.randint(2, 40)) if i % 2 else
              SamplingParams(temperature=0.9, top_k=rng.choice([0, 20]), top_p=1.0, min_p=0.0,
                             seed=70 + i, n_predict=rng.randint(2, 40)) for i in range(n)]

    def run(folder, pipeline, pages):
        eng = Engine(EngineConfig(model=str(folder), dtype="float32", num_pages=pages,
                                  max_batch=6, token_budget=48, chunk=40, pipeline=pipeline))
        out = eng.generate(prompts, params)
        eng.cache.check()
        assert eng.cache.num_free_pages() == pages and eng.cache.num_free_slots == 6
        assert not eng._on_the_way
        return out, eng

    free, _ = run(model_dirs["B"], False, 400)
    # an end-of-sequence token: one that a request draws while others' prompts are under way
    counts = {}
    for o in free:
        for t in o[1:6]:
            counts[t] = counts.get(t, 0) + 1
    eos = max(counts, key=counts.get)
    cfg = json.loads((model_dirs["B"] / "config.json").read_text())
    cfg["eos_token_id"] = eos
    folder = tmp_path / "with_eos"
    folder.mkdir()
    (folder / "config.json").write_text(json.dumps(cfg))
    (folder / "model.safetensors").write_bytes((model_dirs["B"] / "model.safetensors").read_bytes())
    want, _ = run(folder, False, 400)
    assert any(o[-1] == eos and len(o) < p.n_predict for o, p in zip(want, params))
    got, eng = run(folder, True, 400)
    assert got == want
    assert eng.pipelined_steps > 20
    assert sum(r.dropped for r in eng.requests.values()) == 0     # all thrown away by now
    tight, eng = run(folder, True, 26)
    assert tight == want
    assert eng.scheduler.preempted_total > 0 and eng.pipelined_steps > 20


def test_random_workload_with_and_without_graphs(model_dirs):
    """Forty requests of random lengths and options through the scheduler, prompts in portions
    beside decoded tokens: captured graphs, runs of queued decode steps, batches filled up with
    dummy rows and a pool so tight that requests are preempted and computed again must all give
    the tokens of eager steps in a roomy pool (float32, so the arithmetic is the same)."""
    import random
    from kappai_amd.engine import Engine, EngineConfig
    from kappai_amd.sampling import SamplingParams
    rng = random.Random(1)
    vocab = TINY["B"][0]["vocab_size"]
    n = 40
    prompts = [[rng.randrange(vocab) for _ in range(rng.randint(1, 200))] for _ in range(n)]
    params = []
    for i in range(n):
        if rng.random() < 0.5:
            params.append(SamplingParams.greedy(n_predict=rng.randint(1, 60)))
        else:
            params.append(SamplingParams(
                temperature=rng.choice([0.7, 1.0]), top_k=rng.choice([0, 12, 40]),
                top_p=rng.choice([1.0, 0.9]), min_p=rng.choice([0.0, 0.05]), seed=100 + i,
                n_predict=rng.randint(1, 60)))
    results = {}
    for graphs, pages in ((False, 2000), (True, 2000), (True, 90)):
        eng = Engine(EngineConfig(model=str(model_dirs["B"]), dtype="float32", num_pages=pages,
                                  max_batch=16, token_budget=128, chunk=96,
                                  decode_run=8 if graphs else 1, pipeline=graphs))
        eng.runner.decode_graphs = graphs
        results[(graphs, pages)] = eng.generate(prompts, params)
        eng.cache.check()
        assert eng.cache.num_free_pages() == pages and eng.cache.num_free_slots == 16
        assert (eng.scheduler.preempted_total > 0) == (pages == 90)
        assert (eng.runner.graph_replays > 30) == graphs
    assert [len(o) for o in results[(False, 2000)]] == [p.n_predict for p in params]
    assert results[(True, 2000)] == results[(False, 2000)]
    assert results[(True, 90)] == results[(False, 2000)]
