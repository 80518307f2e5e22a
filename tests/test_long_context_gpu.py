"""Contexts of 32,768 and 131,072 tokens: the attention kernels alone against a float32 reference
over the same pages, and a whole narrow model against the plain implementation.

What these lengths reach and shorter tests do not: the cap on the number of key splits of the
decode kernel and the merge over that many partial results, the kernel's own choice of the keys
per split from the lengths of all rows, block tables thousands of pages wide, rotation tables
past 2^16 positions, the single decoded tokens of a step that go to the decode kernel beside
prompt portions at the context length from which the engine really does that, and the tiled
kernels over tens of thousands of cached keys.

Pools are poisoned: pages that no table names hold NaN, and so do the places of a request's last
page beyond its length.  Requests share the random pages of one pool (each through a table in an
order of its own), which keeps the pool small; nothing is stored in these kernel tests."""
import math

import numpy as np
import pytest
import torch

import emulated_ops as ref
from replay_common import make_requests

pytestmark = pytest.mark.gpu

F32, BF16 = torch.float32, torch.bfloat16
DEV = "cuda:0"
BF16_ULP = 2.0 ** -8


@pytest.fixture(scope="module")
def ops():
    from kappai_amd.kernels import ops as real
    return real


def rand(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


def close(got, want, rel, what=""):
    got, want = got.detach().cpu().double(), want.detach().cpu().double()
    assert got.shape == want.shape, (what, got.shape, want.shape)
    assert torch.isfinite(got).all(), what
    scale = max(float(want.abs().max()), 1e-30)
    err = float((got - want).abs().max()) / scale
    assert err <= rel, f"{what}: error {err:.3g} of the largest value, allowed {rel:.3g}"


def shared_pool_case(seed, G, d, ps, lens):
    """Requests holding ``lens`` tokens.  One pool of random pages, enough for the longest;
    every request's table names them in an order of its own, but its last page is one that
    only it has (NaN beyond its length); a tenth more pages that no table names hold NaN."""
    gen = np.random.default_rng(seed)
    S = len(lens)
    blocks = [(n + ps - 1) // ps for n in lens]
    common = max(blocks)
    n_pages = common + S + common // 10 + 1
    k_pool = torch.full((n_pages, G, ps, d), float("nan"), dtype=BF16)
    v_pool = torch.full((n_pages, G, d, ps), float("nan"), dtype=BF16)
    order = gen.permutation(n_pages)
    shared, own = order[:common], order[common:common + S]
    k_pool[torch.from_numpy(shared)] = rand((common, G, ps, d), BF16, seed + 1)
    v_pool[torch.from_numpy(shared)] = rand((common, G, d, ps), BF16, seed + 2)
    bt = np.full((S, common), -1, dtype=np.int32)
    for s in range(S):
        bt[s, :blocks[s] - 1] = gen.permutation(shared)[:blocks[s] - 1]
        bt[s, blocks[s] - 1] = own[s]
        held = lens[s] - (blocks[s] - 1) * ps
        k_pool[own[s], :, :held, :] = rand((G, held, d), BF16, seed + 10 + s)
        v_pool[own[s], :, :, :held] = rand((G, d, held), BF16, seed + 40 + s)
    return k_pool, v_pool, bt


def mark_far_keys(q_row, k_pool, v_pool, bt_row, n, ps, H, G, d, places):
    """Makes head j of the row find the key at ``places[j]`` and nothing else: the head's query
    is 60 in one component (a component of its own per head of a kv head), every key of the
    request is 0 there, and the marked key 8.  Returns the values that must come out."""
    rep = H // G
    want = {}
    pages = torch.from_numpy(bt_row[:(n + ps - 1) // ps].astype(np.int64))
    for j, far in enumerate(places):
        g, comp = j // rep, 3 + 2 * (j % rep)
        q_row[j * d:(j + 1) * d] = 0
        q_row[j * d + comp] = 60.0
        k_pool[pages, g, :, comp] = torch.where(torch.isnan(k_pool[pages, g, :, comp]),
                                                k_pool[pages, g, :, comp],
                                                torch.zeros((), dtype=BF16))
    for j, far in enumerate(places):
        g, comp = j // rep, 3 + 2 * (j % rep)
        k_pool[bt_row[far // ps], g, far % ps, comp] = 8.0
        want[j] = v_pool[bt_row[far // ps], g, :, far % ps].float().clone()
    return want


def decode_split_plan(ops, T, G, d, n_keys):
    """(most splits, planned) as ``ops._decode_split`` and the kernel's launcher settle them."""
    from kappai_amd.kernels.lib import library
    kpw = library("attention_mfma", HEAD_DIM=d).kappai_attn_keys_per_wave()
    _, n_splits = ops.decode_splits(kpw, T, G, n_keys)
    return n_splits, T * G * n_splits > ops.DECODE_WAVES // 2


@pytest.mark.parametrize("n_keys", [32768, 131072])
@pytest.mark.parametrize("rows", ["one row", "sixteen rows"])
def test_decode_attention_at_long_context(ops, n_keys, rows):
    """The decode kernel that splits a row's keys over blocks, and its merge, at context lengths
    where the number of splits is at its cap (one row: the cap alone decides) and where the
    kernel settles the keys per split from all rows' lengths (sixteen rows of mixed lengths).
    Every row against the reference over its own keys; three heads of the longest row each find
    one key only: on the first page, in the middle, on the last page."""
    H, G, d, ps = 4, 2, 64, 16
    if rows == "one row":
        lens = [n_keys]
    else:
        lens = [n_keys, n_keys - 1, n_keys // 2 + 3, 4097, 4096, 513, 100, 1, n_keys - 4000,
                n_keys // 3, 20000, 65, 64, n_keys - 17, 9000, 3]
    T = len(lens)
    n_splits, planned = decode_split_plan(ops, T, G, d, n_keys)
    assert n_splits == ops.DECODE_MAX_SPLITS, "the case is meant to reach the cap on the splits"
    assert planned == (T > 1), "sixteen rows are meant to make the kernel plan its splits"
    k_pool, v_pool, bt = shared_pool_case(3, G, d, ps, lens)
    q = rand((T, H * d), BF16, 5)
    marked = mark_far_keys(q[0], k_pool, v_pool, bt[0], n_keys, ps, H, G, d,
                           [7, n_keys // 2 + 1, n_keys - 2])
    row_pos = torch.tensor([n - 1 for n in lens], dtype=torch.int32)
    row_seg = torch.arange(T, dtype=torch.int32)
    scale = 1.0 / math.sqrt(d)
    want = ref.paged_attention(q.float(), H, G, d, k_pool.float(), v_pool.float(), row_pos,
                               row_seg, torch.from_numpy(bt), ps, scale)
    got = ops.paged_attention(q.to(DEV), H, G, d, k_pool.to(DEV), v_pool.to(DEV), row_pos.to(DEV),
                              row_seg.to(DEV), torch.from_numpy(bt).to(DEV), ps, scale,
                              single_rows=True, max_position=n_keys - 1, kernel="decode-split")
    close(got.float(), want, 2 * BF16_ULP, f"decode attention over {n_keys} keys, {rows}")
    for j, value in marked.items():
        close(got[0, j * d:(j + 1) * d].float(), value, 2 * BF16_ULP, f"far key of head {j}")


@pytest.mark.parametrize("n_keys", [32768, 131072])
def test_decode_attention_with_a_window_edge_far_out(ops, n_keys):
    """A window of 5,000 keys over contexts of up to ``n_keys``: the window's first key lies far
    beyond the first pages.  Head 0 of the longest row finds the first key inside the window; head
    1's only matching key lies one place outside it and must not be seen (its output is then the
    mean of the values inside, as the reference's)."""
    H, G, d, ps, window = 4, 2, 64, 16, 5000
    lens = [n_keys, 5000, 5001, n_keys - 3000, 4999, 70, n_keys // 2, 12000]
    T = len(lens)
    k_pool, v_pool, bt = shared_pool_case(4, G, d, ps, lens)
    q = rand((T, H * d), BF16, 6)
    marked = mark_far_keys(q[0], k_pool, v_pool, bt[0], n_keys, ps, H, G, d,
                           [n_keys - window, n_keys - window - 1])
    row_pos = torch.tensor([n - 1 for n in lens], dtype=torch.int32)
    row_seg = torch.arange(T, dtype=torch.int32)
    scale = 1.0 / math.sqrt(d)
    want = ref.paged_attention(q.float(), H, G, d, k_pool.float(), v_pool.float(), row_pos,
                               row_seg, torch.from_numpy(bt), ps, scale, window=window)
    got = ops.paged_attention(q.to(DEV), H, G, d, k_pool.to(DEV), v_pool.to(DEV), row_pos.to(DEV),
                              row_seg.to(DEV), torch.from_numpy(bt).to(DEV), ps, scale,
                              window=window, single_rows=True, max_position=n_keys - 1,
                              kernel="decode-split")
    close(got.float(), want, 2 * BF16_ULP, f"window of {window} over {n_keys} keys")
    close(got[0, :d].float(), marked[0], 2 * BF16_ULP, "the first key inside the window")
    outside = marked[1]
    assert float((got[0, d:2 * d].float().cpu() - outside).abs().max()) > 0.5, \
        "a key outside the window was seen"


def portion_reference(q, H, G, d, keys, vals, pos0, scale, window=0):
    """Attention of the rows of one portion, whose first row stands at ``pos0``, over the
    request's keys and values [n, G, d] in float32 (the portion's own included): whole matrices
    in place of the reference's row by row, for portions of hundreds of rows over tens of
    thousands of keys."""
    R = q.shape[0]
    n = keys.shape[0]
    out = torch.empty((R, H * d), dtype=F32)
    key_at = torch.arange(n)[None, :]
    row_at = (pos0 + torch.arange(R))[:, None]
    seen = key_at <= row_at
    if window:
        seen &= key_at > row_at - window
    for h in range(H):
        g = h // (H // G)
        sc = (q[:, h * d:(h + 1) * d].float() @ keys[:, g, :].T) * scale
        sc = sc.masked_fill(~seen, float("-inf"))
        out[:, h * d:(h + 1) * d] = torch.softmax(sc, dim=1) @ vals[:, g, :]
    return out


@pytest.mark.parametrize("n_keys,new", [(32768, 256), (131072, 96)])
@pytest.mark.parametrize("variant", [1, 2])
@pytest.mark.parametrize("window", [0, 4500])
def test_prefill_attention_after_a_long_history(ops, n_keys, new, variant, window):
    """A prompt portion whose request already holds tens of thousands of keys, through both forms
    of the tiled kernel (2: key tiles shared by four query heads through LDS), without and with a
    window whose edge lies far out.  One head of the last row finds a single far key; with a
    window, a second head's only matching key lies just outside it."""
    H, G, d, ps = 8, 2, 64, 16
    k_pool, v_pool, bt = shared_pool_case(8, G, d, ps, [n_keys])
    q = rand((new, H * d), BF16, 9)
    first_seen = n_keys - window if window else 0
    places = [first_seen + 2] + ([first_seen - 1] if window else [n_keys // 2])
    marked = mark_far_keys(q[new - 1], k_pool, v_pool, bt[0], n_keys, ps, H, G, d, places)
    pos0 = n_keys - new
    row_pos = torch.arange(pos0, n_keys, dtype=torch.int32)
    row_seg = torch.zeros(new, dtype=torch.int32)
    nt = (new + 31) // 32
    tiles = torch.tensor([(0, r, min(32, new - r), j | (nt << 16))
                          for j, r in enumerate(range(0, new, 32))], dtype=torch.int32)
    pages = torch.from_numpy(bt[0].astype(np.int64))
    keys = k_pool[pages].float().permute(0, 2, 1, 3).reshape(-1, G, d)[:n_keys]
    vals = v_pool[pages].float().permute(0, 3, 1, 2).reshape(-1, G, d)[:n_keys]
    scale = 1.0 / math.sqrt(d)
    want = portion_reference(q, H, G, d, keys, vals, pos0, scale, window)
    got = ops.paged_attention(q.to(DEV), H, G, d, k_pool.to(DEV), v_pool.to(DEV), row_pos.to(DEV),
                              row_seg.to(DEV), torch.from_numpy(bt).to(DEV), ps, scale,
                              window=window, q_tiles=tiles.to(DEV), kernel="prefill",
                              max_position=n_keys - 1, prefill_variant=variant)
    close(got.float(), want, 2 * BF16_ULP, f"{new} rows after {pos0} keys, form {variant}")
    close(got[new - 1, :d].float(), marked[0], 2 * BF16_ULP, "the far key")
    if window:
        assert float((got[new - 1, d:2 * d].float().cpu() - marked[1]).abs().max()) > 0.5, \
            "a key outside the window was seen"
    else:
        close(got[new - 1, d:2 * d].float(), marked[1], 2 * BF16_ULP, "the far key in the middle")


@pytest.mark.parametrize("n_keys", [32768, 131072])
def test_lone_rows_beside_a_portion_at_long_context(ops, n_keys):
    """Three single decoded tokens over 4,096 to ``n_keys`` keys beside a prompt portion of 70
    rows: the single rows go through the decode kernel by a list (``lone_rows``), the portion
    through the tiled kernel.  The longest row finds far keys on its first page, in the middle
    and on its last page."""
    H, G, d, ps = 4, 2, 64, 16
    lens = [70, n_keys, 4096, n_keys // 2 + 9]
    new = [70, 1, 1, 1]
    k_pool, v_pool, bt = shared_pool_case(12, G, d, ps, lens)
    T = sum(new)
    q = rand((T, H * d), BF16, 13)
    marked = mark_far_keys(q[70], k_pool, v_pool, bt[1], n_keys, ps, H, G, d,
                           [3, n_keys // 2, n_keys - 1])
    row_seg = torch.tensor([0] * 70 + [1, 2, 3], dtype=torch.int32)
    row_pos = torch.tensor(list(range(70)) + [n - 1 for n in lens[1:]], dtype=torch.int32)
    tiles = torch.tensor([(0, 0, 32, 0 | (3 << 16)), (0, 32, 32, 1 | (3 << 16)),
                          (0, 64, 6, 2 | (3 << 16))], dtype=torch.int32)
    lone = torch.tensor([70, 71, 72], dtype=torch.int32)
    scale = 1.0 / math.sqrt(d)
    want = ref.paged_attention(q.float(), H, G, d, k_pool.float(), v_pool.float(), row_pos,
                               row_seg, torch.from_numpy(bt), ps, scale)
    got = ops.paged_attention(q.to(DEV), H, G, d, k_pool.to(DEV), v_pool.to(DEV), row_pos.to(DEV),
                              row_seg.to(DEV), torch.from_numpy(bt).to(DEV), ps, scale,
                              q_tiles=tiles.to(DEV), kernel="prefill", max_position=n_keys - 1,
                              lone_rows=lone.to(DEV), max_lone_position=n_keys - 1)
    close(got.float(), want, 2 * BF16_ULP, f"lone rows over up to {n_keys} keys")
    for j, value in marked.items():
        close(got[70, j * d:(j + 1) * d].float(), value, 2 * BF16_ULP, f"far key of head {j}")


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_rotation_and_store_at_positions_past_two_to_the_sixteenth(ops, dtype):
    """Per-head norm, rotation and the store into the pages for rows at positions around 65,536
    and 131,071: the rotation tables are as long, the block tables 8,192 pages wide."""
    H, G, d, ps = 4, 2, 64, 16
    positions = [65535, 65536, 65537, 100000, 131070, 131071]
    T = len(positions)
    width = 131072 // ps
    gen = np.random.default_rng(2)
    n_pages = 64
    bt = np.full((T, width), -1, dtype=np.int32)
    own = gen.permutation(n_pages)[:T]
    for t, p in enumerate(positions):
        bt[t, p // ps] = own[t]
    qkv = rand((T, (H + 2 * G) * d), dtype, 3)
    qn, kn = 1 + rand((d,), F32, 4, 0.2), 1 + rand((d,), F32, 5, 0.2)
    half = d // 2
    freq = np.power(1e6, -2.0 * np.arange(half) / d)
    ang = np.arange(131072)[:, None] * freq[None, :]
    cos, sin = (torch.from_numpy(np.cos(ang).astype(np.float32)),
                torch.from_numpy(np.sin(ang).astype(np.float32)))
    k_pool = torch.full((n_pages, G, ps, d), float("nan"), dtype=dtype)
    v_pool = torch.full((n_pages, G, d, ps), float("nan"), dtype=dtype)
    row_pos = torch.tensor(positions, dtype=torch.int32)
    row_seg = torch.arange(T, dtype=torch.int32)
    dev_qkv, dev_k, dev_v = qkv.to(DEV), k_pool.to(DEV), v_pool.to(DEV)
    ops.qk_norm_rope_store(dev_qkv, H, G, d, qn.to(DEV), kn.to(DEV), 1e-5, cos.to(DEV),
                           sin.to(DEV), d, 1, dev_k, dev_v, row_pos.to(DEV), row_seg.to(DEV),
                           torch.from_numpy(bt).to(DEV), ps)
    qkv_ref, k_ref, v_ref = qkv.float(), k_pool.float(), v_pool.float()
    ref.qk_norm_rope_store(qkv_ref, H, G, d, qn, kn, 1e-5, cos, sin, d, 1, k_ref, v_ref, row_pos,
                           row_seg, torch.from_numpy(bt), ps)
    tol = BF16_ULP if dtype == BF16 else 3e-6
    close(dev_qkv[:, :H * d].float(), qkv_ref[:, :H * d], tol, "q")
    assert torch.equal(~torch.isnan(k_ref), ~torch.isnan(dev_k.cpu().float())), "other places"
    close(torch.nan_to_num(dev_k.float()), torch.nan_to_num(k_ref), tol, "k pages")
    close(torch.nan_to_num(dev_v.float()), torch.nan_to_num(v_ref), 0.0, "v pages")


# ---------------------------------------------------------------------------------------------
# the whole model
# ---------------------------------------------------------------------------------------------
LONG_MODEL = {
    "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2",
    "hidden_size": 128, "num_hidden_layers": 3,
    "layer_types": ["conv", "full_attention", "conv"],
    "num_attention_heads": 16, "num_key_value_heads": 4, "head_dim": 64,
    "intermediate_size": 256, "block_auto_adjust_ff_dim": False,
    "vocab_size": 512, "norm_eps": 1e-5, "rope_theta": 1000000.0,
    "conv_L_cache": 3, "conv_bias": False, "tie_embedding": True,
    "max_position_embeddings": 40000,
}
LONG_PROMPT, LONG_PORTION, LONG_TAIL = 32768, 2048, 32


@pytest.fixture(scope="module")
def long_model(tmp_path_factory):
    import copy
    from kappai_amd.config import config_from_dict
    from kappai_amd.weights import write_random_model
    folder = tmp_path_factory.mktemp("long") / "model"
    return write_random_model(folder, config_from_dict(copy.deepcopy(LONG_MODEL)), seed=8,
                              std=0.05, norm_jitter=0.1)


_long_plain = {}


def long_plain_logits(model_dir, requests, wanted, rounded):
    """The plain implementation's logits at the wanted (id, position) only."""
    from plain import lfm2 as plain
    key = (str(model_dir), rounded)
    if key not in _long_plain:
        cfg, w = plain.read_model_dir(model_dir)
        kw = {"rnd": plain.round_bf16} if rounded else {}
        out = {}
        for rid, toks in requests.items():
            rows = sorted(pos for r, pos in wanted if r == rid)
            out[rid] = plain.forward(cfg, w, toks, rows=rows, **kw)
        _long_plain[key] = out
    return _long_plain[key]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_prompt_of_32k_tokens_beside_decoding_requests(tmp_path, long_model, dtype):
    """One request's prompt of 32,768 tokens in portions of 2,048 beside two requests that decode
    (one of them over more than 4,096 keys, so that in every such step its single row leaves the
    tiles for the decode kernel), then 32 tokens one by one for all three, from a pool that the
    requests fill.  The logits at the last row of every portion, and at every decoded token of
    the three, against the plain implementation.  The state of the conv layers and the keys are
    handed from portion to portion as in kappai's src/test/test_hybrid.c:164-215 (150 tokens = 3 x
    50 = 64 + 64 + 22) and :305-353 (a prompt, then greedy steps), at a length where every portion
    after the first few reads tens of thousands of cached keys."""
    import schedules
    from kappai_amd.engine.replay import TraceReplayer, make_replay_cache
    from kappai_amd.engine.step import StepRunner
    from kappai_amd.kernels import tuning
    from kappai_amd.models import load_model
    import replay_common

    n_portions = LONG_PROMPT // LONG_PORTION
    lengths = {"long": LONG_PROMPT + LONG_TAIL, "mid": 4200 + n_portions + LONG_TAIL,
               "short": 50 + n_portions + LONG_TAIL}
    assert tuning.LONE_ROWS_FROM and 4200 >= tuning.LONE_ROWS_FROM
    requests = make_requests(LONG_MODEL["vocab_size"], list(lengths.values()), seed=77)
    requests = dict(zip(lengths, requests.values()))
    plans = {"mid": (0, [4200] + [1] * (n_portions + LONG_TAIL)),
             "short": (0, [50] + [1] * (n_portions + LONG_TAIL)),
             "long": (1, [LONG_PORTION] * n_portions + [1] * LONG_TAIL)}
    steps, index, peak = schedules.build(requests, plans, want="last")
    model = load_model(long_model, dtype, DEV)
    cache = make_replay_cache(model, peak)
    cache.allocate_storage(model.dtype, DEV, poison=True)
    runner = StepRunner(model, cache, DEV)
    rep = TraceReplayer(runner, tmp_path / "out")
    outputs = {}
    for obj in steps:
        res = rep.run_step(obj)
        if res is not None:
            outputs[obj["step"]] = res
    cache.check()
    assert not cache.live_requests()
    if dtype == "bfloat16":
        assert runner.graph_replays >= LONG_TAIL - 3      # the last steps ran from graphs
    got = replay_common.collect(index, outputs, model.vocab_size)
    assert len(got) == sum(len(p) for _, p in plans.values())
    wanted = list(got)
    ref_logits = long_plain_logits(long_model, requests, wanted, rounded=False)
    scale = max(float(np.nanmax(np.abs(v))) for v in ref_logits.values())
    errs = {k: float(np.abs(row.astype(np.float64) - ref_logits[k[0]][k[1]]).max()) / scale
            for k, row in got.items()}
    worst = max(errs, key=errs.get)
    if dtype == "float32":
        assert errs[worst] < replay_common.FP32_TOL, (worst, errs[worst])
        return
    rounded = long_plain_logits(long_model, requests, wanted, rounded=True)
    own = {k: float(np.abs(rounded[k[0]][k[1]] - ref_logits[k[0]][k[1]]).max()) / scale
           for k in wanted}
    assert errs[worst] < replay_common.BF16_MAX_FACTOR * max(own.values()), (
        worst, errs[worst], max(own.values()))
    rms = math.sqrt(sum(float(((row.astype(np.float64) - ref_logits[k[0]][k[1]]) ** 2).sum())
                        for k, row in got.items()) / (len(got) * model.vocab_size)) / scale
    rms_own = math.sqrt(sum(float(((rounded[k[0]][k[1]] - ref_logits[k[0]][k[1]]) ** 2).sum())
                            for k in wanted) / (len(wanted) * model.vocab_size)) / scale
    assert rms < replay_common.BF16_RMS_FACTOR * rms_own, (rms, rms_own)
