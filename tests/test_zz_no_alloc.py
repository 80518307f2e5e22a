"""The decode attention's entry point that allocates nothing (``kappai_attn_decode_static``,
``csrc/no_alloc.h``), called through ctypes: it keeps the splits' partial results in a device
array of the library's own and must give, bit for bit, what ``kappai_attn_decode`` gives with a
workspace from the caller, also on a second call with a smaller input, which finds the first
call's partial results still in the array.  That it allocates nothing is checked twice: the
driver's count of free device memory does not move across the call, and the call can be recorded
into a HIP graph, where an allocation is an error."""
import ctypes
import math

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
c_int, c_float, vp = ctypes.c_int, ctypes.c_float, ctypes.c_void_p


def decode_case(seed, T, H, G, d, ps, lengths):
    """T requests that hold ``lengths`` keys each (the row's own included) in shuffled pages."""
    g = torch.Generator().manual_seed(seed)
    blocks = [(n + ps - 1) // ps for n in lengths]
    n_pages = sum(blocks) + 2
    perm = torch.randperm(n_pages, generator=g).tolist()
    bt = np.full((T, max(blocks)), -1, dtype=np.int32)
    k = 0
    for s in range(T):
        for b in range(blocks[s]):
            bt[s, b] = perm[k]
            k += 1
    q = (torch.randn((T, H * d), generator=g) * 1.5).to(torch.bfloat16)
    k_pool = torch.randn((n_pages, G, ps, d), generator=g).to(torch.bfloat16)
    v_pool = torch.randn((n_pages, G, d, ps), generator=g).to(torch.bfloat16)
    return dict(q=q.to(DEV), k_pool=k_pool.to(DEV), v_pool=v_pool.to(DEV),
                row_pos=torch.tensor([n - 1 for n in lengths], dtype=torch.int32, device=DEV),
                row_seg=torch.arange(T, dtype=torch.int32, device=DEV),
                bt=torch.from_numpy(bt).to(DEV))


def run_both(lib, case, T, H, G, d, ps, keys_per_split, n_splits):
    stream = vp(torch.cuda.current_stream().cuda_stream)
    scale = c_float(1.0 / math.sqrt(d))
    common = lambda out: (vp(case["q"].data_ptr()), c_int(case["q"].stride(0)),        # noqa: E731
                          vp(case["k_pool"].data_ptr()), vp(case["v_pool"].data_ptr()),
                          vp(out.data_ptr()), c_int(H * d))
    tables = (vp(case["row_pos"].data_ptr()), vp(case["row_seg"].data_ptr()),
              vp(case["bt"].data_ptr()), c_int(case["bt"].shape[1]), c_int(T), c_int(H), c_int(G),
              c_int(ps), c_int(0), scale, c_int(keys_per_split), c_int(n_splits), stream)
    want = torch.full((T, H * d), float("nan"), dtype=torch.bfloat16, device=DEV)
    part_o = torch.empty((T, H, n_splits, d), dtype=torch.float32, device=DEV)
    part_ml = torch.empty((T, H, n_splits, 2), dtype=torch.float32, device=DEV)
    rc = lib.kappai_attn_decode(*common(want), vp(part_o.data_ptr()), vp(part_ml.data_ptr()),
                                *tables)
    assert rc == 0, rc
    got = torch.full((T, H * d), float("nan"), dtype=torch.bfloat16, device=DEV)
    torch.cuda.synchronize()
    # the driver's own count of free bytes (torch's allocator counter would not see a hipMalloc
    # inside the library); the array's address was looked up before (init), so nothing is left
    # that the call may take
    free_before = torch.cuda.mem_get_info(DEV)[0]
    rc = lib.kappai_attn_decode_static(*common(got), *tables)
    assert rc == 0, (rc, lib.kappai_attn_decode_static_error().decode())
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info(DEV)[0] == free_before
    return got.cpu(), want.cpu()


def capture_static(lib, case, T, H, G, d, ps, keys_per_split, n_splits, replays=3):
    """The same call recorded into a HIP graph: while a stream is being captured (torch captures
    in the mode that forbids it on every thread) a hipMalloc or hipFree fails and ends the
    capture with an error, so a call that allocates and frees again is caught here where the
    count of free bytes would not show it.  Returns the output of every replay."""
    scale = c_float(1.0 / math.sqrt(d))
    out = torch.full((T, H * d), float("nan"), dtype=torch.bfloat16, device=DEV)
    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.graph(graph):
        rc = lib.kappai_attn_decode_static(
            vp(case["q"].data_ptr()), c_int(case["q"].stride(0)), vp(case["k_pool"].data_ptr()),
            vp(case["v_pool"].data_ptr()), vp(out.data_ptr()), c_int(H * d),
            vp(case["row_pos"].data_ptr()), vp(case["row_seg"].data_ptr()),
            vp(case["bt"].data_ptr()), c_int(case["bt"].shape[1]), c_int(T), c_int(H), c_int(G),
            c_int(ps), c_int(0), scale, c_int(keys_per_split), c_int(n_splits),
            vp(torch.cuda.current_stream().cuda_stream))
    assert rc == 0, (rc, lib.kappai_attn_decode_static_error().decode())
    outs = []
    for _ in range(replays):
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        outs.append(out.cpu().clone())
    return outs


@pytest.mark.parametrize("d", [64, 128])
def test_static_decode_matches_the_workspace_form_twice(d):
    from kappai_amd.kernels.lib import library

    lib = library("attention_mfma", HEAD_DIM=d)
    lib.kappai_attn_decode_static_error.restype = ctypes.c_char_p
    assert lib.kappai_attn_decode_static_init() == 0
    kpw = lib.kappai_attn_keys_per_wave()
    H, G, ps = 8, 2, 16
    # the larger input first, then a smaller one that finds the first one's partial results in
    # the array: fewer rows, fewer splits, shorter requests
    for seed, lengths, n_splits in ((1, [700, 33, 1, 512, 129, 1000], 8), (2, [40, 300, 2], 3)):
        T = len(lengths)
        n_keys = max(lengths)
        keys_per_split = ((n_keys + n_splits - 1) // n_splits + kpw - 1) // kpw * kpw
        n_splits = (n_keys + keys_per_split - 1) // keys_per_split
        case = decode_case(seed, T, H, G, d, ps, lengths)
        got, want = run_both(lib, case, T, H, G, d, ps, keys_per_split, n_splits)
        assert not torch.isnan(want.float()).any()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), (d, lengths)
        for replayed in capture_static(lib, case, T, H, G, d, ps, keys_per_split, n_splits):
            assert torch.equal(replayed.view(torch.int16), want.view(torch.int16)), (d, lengths)


def test_static_decode_refuses_what_its_array_cannot_hold():
    from kappai_amd.kernels.lib import library

    d = 64
    lib = library("attention_mfma", HEAD_DIM=d)
    lib.kappai_attn_decode_static_error.restype = ctypes.c_char_p
    cap = lib.kappai_attn_decode_static_capacity()
    kpw = lib.kappai_attn_keys_per_wave()
    H, G, ps, T = 32, 8, 16, 64
    n_splits = cap // (T * H * (d + 2)) + 1
    case = decode_case(3, T, H, G, d, ps, [n_splits * kpw] * T)
    out = torch.zeros((T, H * d), dtype=torch.bfloat16, device=DEV)
    rc = lib.kappai_attn_decode_static(
        vp(case["q"].data_ptr()), c_int(H * d), vp(case["k_pool"].data_ptr()),
        vp(case["v_pool"].data_ptr()), vp(out.data_ptr()), c_int(H * d),
        vp(case["row_pos"].data_ptr()), vp(case["row_seg"].data_ptr()), vp(case["bt"].data_ptr()),
        c_int(case["bt"].shape[1]), c_int(T), c_int(H), c_int(G), c_int(ps), c_int(0),
        c_float(0.125), c_int(kpw), c_int(n_splits),
        vp(torch.cuda.current_stream().cuda_stream))
    assert rc != 0
    msg = lib.kappai_attn_decode_static_error().decode()
    assert "floats of partial results" in msg and str(cap) in msg, msg
    torch.cuda.synchronize()
    assert not out.any()          # nothing ran
