"""Each HIP kernel alone against a plain torch reference of the same operation (the CPU
stand-ins of emulated_ops.py, or float64 torch), at sizes other than the engine's."""
import math

import numpy as np
import pytest
import torch

import emulated_ops as ref

pytestmark = pytest.mark.gpu

F32, BF16 = torch.float32, torch.bfloat16
DEV = "cuda:0"


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


BF16_ULP = 2.0 ** -8      # half a unit in the last place of a bfloat16 is 2^-9 of its value


# ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [F32, BF16])
def test_embed_rows(ops, dtype):
    table = rand((1000, 200), dtype, 1)
    ids = torch.tensor([0, 999, 5, 5, 17, 123, 998], dtype=torch.int32)
    got = ops.embed_rows(ids.to(DEV), table.to(DEV))
    assert got.dtype == F32
    assert torch.equal(got.cpu(), table[ids.long()].float())


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("D", [96, 1000, 2048, 4104])
def test_embedding_and_first_norm_in_one_kernel(ops, dtype, D):
    """The kernel that embeds and normalises gives the bits of the two kernels it stands for: from
    float rows, bfloat16 rows and a bfloat16 table kept in fragment order, as plain rows and as
    rows in fragment order."""
    V = 208
    w = (1 + rand((D,), F32, 4, 0.2)).to(DEV)
    tables = [rand((V, D), F32, 1).to(DEV), rand((V, D), BF16, 2).to(DEV)]
    if D % 32 == 0:
        tables.append(ops.InFragments.of(tables[1]))
    for T in (1, 7, 13, 40):
        ids = torch.randint(0, V, (T,), generator=torch.Generator().manual_seed(T)).int().to(DEV)
        for table in tables:
            for fragment in (False, True):
                if fragment and not ops.FragmentRows.fits(T, D, dtype):
                    continue
                want_resid = ops.embed_rows(ids, table)
                want = ops.add_rmsnorm(want_resid.clone(), None, w, 1e-5, dtype, fragment=fragment)
                resid, got = ops.embed_rmsnorm(ids, table, w, 1e-5, dtype, fragment=fragment)
                assert torch.equal(resid, want_resid)
                if fragment:
                    got, want = got.materialize(), want.materialize()
                assert torch.equal(got, want), (T, D, fragment, type(table).__name__)
    with pytest.raises(ValueError):
        ops.embed_rmsnorm(ids, rand((V, 100), BF16, 3).to(DEV), w[:100].contiguous(), 1e-5, dtype)


def test_stream_read_stays_inside_the_buffer(ops):
    """The read-only yardstick kernel reads whole pieces of 32 KB for each of its 512 blocks and
    never more than the buffer holds; a buffer too small for one piece a block is refused."""
    for n_bytes in (16 << 20, (16 << 20) + 12345 * 16, 100 * 1000 * 1000):
        buf = torch.zeros(n_bytes // 4, dtype=torch.int32, device=DEV)
        got = ops.stream_read(buf)
        assert 0 < got <= n_bytes and got % (512 * 32768) == 0 and n_bytes - got < 512 * 32768
        for blocks in (256, 2048):
            if n_bytes < blocks * 32768:          # not one piece a block: refused (below)
                continue
            got = ops.stream_read(buf, blocks=blocks)
            assert 0 < got <= n_bytes and got % (blocks * 32768) == 0
            assert n_bytes - got < blocks * 32768
    torch.cuda.synchronize()
    with pytest.raises(RuntimeError):
        ops.stream_read(torch.zeros(1000, dtype=torch.int32, device=DEV))


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("D", [64, 96, 1000, 2048, 5000])
def test_add_rmsnorm(ops, dtype, D):
    T = 13
    resid = rand((T, D), F32, 2, 3.0)
    delta = rand((T, D), dtype, 3)
    w = 1 + rand((D,), F32, 4, 0.2)
    for eps in (1e-5, 1e-2):
        r_dev = resid.to(DEV).clone()
        got = ops.add_rmsnorm(r_dev, delta.to(DEV), w.to(DEV), eps, dtype)
        r_ref = resid.clone()
        want = ref.add_rmsnorm(r_ref, delta, w, eps, F32)
        close(got.float(), want, BF16_ULP if dtype == BF16 else 2e-6, "normed")
        close(r_dev, r_ref, 1e-7, "residual")
    # no delta; row selection leaves the residual alone
    rows = torch.tensor([12, 0, 5], dtype=torch.int32)
    r_dev = resid.to(DEV).clone()
    got = ops.add_rmsnorm(r_dev, delta.to(DEV), w.to(DEV), 1e-6, dtype, rows=rows.to(DEV),
                          write_resid=False)
    want = ref.add_rmsnorm(resid.clone(), delta, w, 1e-6, F32, rows=rows, write_resid=False)
    close(got.float(), want, BF16_ULP if dtype == BF16 else 2e-6, "selected rows")
    assert torch.equal(r_dev.cpu(), resid)
    got = ops.add_rmsnorm(r_dev, None, w.to(DEV), 1e-6, dtype)
    close(got.float(), ref.add_rmsnorm(resid.clone(), None, w, 1e-6, F32),
          BF16_ULP if dtype == BF16 else 2e-6, "no delta")


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_swiglu(ops, dtype):
    gu = rand((9, 2 * 333), dtype, 5, 2.0)
    got = ops.swiglu(gu.to(DEV))
    want = ref.swiglu(gu.float())
    close(got.float(), want, BF16_ULP if dtype == BF16 else 2e-6, "swiglu")
    z = torch.zeros((2, 8), dtype=dtype)
    assert float(ops.swiglu(z.to(DEV)).abs().max()) == 0.0


# ---------------------------------------------------------------------------------------
GEMM_SHAPES = [(1, 64, 64), (7, 100, 72), (16, 33, 136), (17, 257, 320), (64, 2048, 96),
               (65, 96, 320), (130, 257, 136), (200, 1000, 2048), (3, 16, 8)]


@pytest.mark.parametrize("M,N,K", GEMM_SHAPES)
def test_linear_float32(ops, M, N, K):
    x, w, b = rand((M, K), F32, 6), rand((N, K), F32, 7), rand((N,), F32, 8)
    want = x.double() @ w.double().T
    close(ops.linear(x.to(DEV), w.to(DEV)), want, 3e-6, "no bias")
    close(ops.linear(x.to(DEV), w.to(DEV), b.to(DEV)), want + b.double(), 3e-6, "bias")
    # a row's result does not depend on what else is in the batch
    if M > 1:
        one = ops.linear(x[:1].to(DEV).contiguous(), w.to(DEV))
        assert torch.equal(one, ops.linear(x.to(DEV), w.to(DEV))[:1])


def test_linear_float32_is_not_reduced_precision(ops):
    """Inputs that differ only below bfloat16/tf32 precision must give different results."""
    K = 8
    x = torch.full((1, K), 1.0 + 2.0 ** -12, dtype=F32)
    w = torch.full((1, K), 1.0 + 2.0 ** -12, dtype=F32)
    got = float(ops.linear(x.to(DEV), w.to(DEV))[0, 0])
    assert abs(got - K * (1.0 + 2.0 ** -12) ** 2) < 4e-6 and got != float(K)


@pytest.mark.parametrize("M,N,K", GEMM_SHAPES + [(33, 130, 72), (48, 6144, 2048), (128, 128, 32),
                                                 (40, 16392, 256), (64, 16384, 128), (32, 16384, 128),
                                                 (513, 640, 264), (2048, 3200, 96),
                                                 (1999, 3330, 40)])
@pytest.mark.parametrize("out_dtype", [F32, BF16])
def test_linear_bfloat16(ops, M, N, K, out_dtype):
    x, w, b = rand((M, K), BF16, 9), rand((N, K), BF16, 10), rand((N,), F32, 11)
    want = x.double() @ w.double().T
    tol = 2e-5 if out_dtype == F32 else BF16_ULP
    for force in ([0, 1, 2] if M <= 64 else [0]):
        got = ops.linear(x.to(DEV), w.to(DEV), out_dtype=out_dtype, force_kernel=force)
        assert got.dtype == out_dtype
        close(got.float(), want, tol, f"kernel {force}")
        got = ops.linear(x.to(DEV), w.to(DEV), b.to(DEV), out_dtype=out_dtype, force_kernel=force)
        close(got.float(), want + b.double(), tol, f"kernel {force} with bias")


@pytest.mark.parametrize("M,F,K", [(1, 16, 64), (8, 192, 64), (16, 320, 96), (33, 208, 120),
                                   (64, 8192, 2048), (65, 320, 96), (200, 1008, 256),
                                   (2048, 1616, 72)])
def test_linear_swiglu(ops, M, F, K):
    x, wg, wu = rand((M, K), BF16, 16), rand((F, K), BF16, 17, 0.2), rand((F, K), BF16, 18, 0.2)
    w = ops.interleave_gate_up(wg.to(DEV), wu.to(DEV))
    assert torch.equal(w.cpu(), ref.interleave_gate_up(wg, wu))
    g, u = x.double() @ wg.double().T, x.double() @ wu.double().T
    want = g / (1 + torch.exp(-g)) * u
    for force in ([0, 1, 2] if M <= 64 else [0]):
        got = ops.linear_swiglu(x.to(DEV), w, force_kernel=force)
        close(got.float(), want, BF16_ULP, f"kernel {force}")


BLOCK256 = 7          # force_kernel: 256 x 256 blocks, one wave a SIMD
BLOCK128 = 8          # the same kernel with 128 x 128 blocks
BLOCK128_DEEP = 10    # 128 x 128 blocks with four LDS buffers (tiles 0-2 loaded ahead)
BLOCK192 = 11         # blocks of 256 rows x 192 columns


@pytest.mark.parametrize("M,N,K", [(256, 256, 128), (300, 520, 256), (129, 8, 128), (1000, 1096, 384),
                                   (2048, 2048, 2048), (513, 264, 1280)])
@pytest.mark.parametrize("out_dtype", [F32, BF16])
@pytest.mark.parametrize("block", [BLOCK256, BLOCK128, BLOCK128_DEEP, BLOCK192])
def test_linear_block256(ops, M, N, K, out_dtype, block):
    """The large-product kernel at sizes that end inside its 256 x 256 blocks, with a row stride
    on the input, with bias, and against the other tiled kernel on the same data."""
    wide = rand((M, K + 24), BF16, 41)
    x, w, b = wide[:, :K], rand((N, K), BF16, 42), rand((N,), F32, 43)
    want = x.double() @ w.double().T
    tol = 2e-5 if out_dtype == F32 else BF16_ULP
    xd = wide.to(DEV)[:, :K]
    got = ops.linear(xd, w.to(DEV), out_dtype=out_dtype, force_kernel=block)
    close(got.float(), want, tol, "block256")
    got = ops.linear(xd, w.to(DEV), b.to(DEV), out_dtype=out_dtype, force_kernel=block)
    close(got.float(), want + b.double(), tol, "block256 with bias")
    other = ops.linear(xd, w.to(DEV), b.to(DEV), out_dtype=out_dtype, force_kernel=5)
    close(got.float(), other.float(), tol, "against 256 x 128 blocks")


@pytest.mark.parametrize("M,F,K", [(256, 128, 128), (300, 1008, 256), (2048, 1616, 384)])
@pytest.mark.parametrize("block", [BLOCK256, BLOCK128, BLOCK128_DEEP])
def test_linear_swiglu_block256(ops, M, F, K, block):
    x, wg, wu = rand((M, K), BF16, 44), rand((F, K), BF16, 45, 0.2), rand((F, K), BF16, 46, 0.2)
    w = ops.interleave_gate_up(wg.to(DEV), wu.to(DEV))
    g, u = x.double() @ wg.double().T, x.double() @ wu.double().T
    want = g / (1 + torch.exp(-g)) * u
    got = ops.linear_swiglu(x.to(DEV), w, force_kernel=block)
    close(got.float(), want, BF16_ULP, "block256")


SHARED_ROWS = 9       # force_kernel: 17 to 64 rows, the rows shared through LDS


@pytest.mark.parametrize("M", [17, 32, 33, 47, 64])
@pytest.mark.parametrize("N,K", [(64, 512), (200, 1024), (2048, 2048), (8200, 1536)])
@pytest.mark.parametrize("out_dtype", [F32, BF16])
def test_linear_shared_rows(ops, M, N, K, out_dtype):
    """The kernel for 17 to 64 rows: every row-tile count, matrices that end inside a block's 64
    columns or inside a wave's 32, one and several chunks of K per wave, a row stride, bias."""
    wide = rand((M, K + 8), BF16, 51)
    x, w, b = wide[:, :K], rand((N, K), BF16, 52), rand((N,), F32, 53)
    want = x.double() @ w.double().T
    tol = 2e-5 if out_dtype == F32 else BF16_ULP
    xd = wide.to(DEV)[:, :K]
    got = ops.linear(xd, w.to(DEV), out_dtype=out_dtype, force_kernel=SHARED_ROWS)
    close(got.float(), want, tol, "shared rows")
    got = ops.linear(xd, w.to(DEV), b.to(DEV), out_dtype=out_dtype, force_kernel=SHARED_ROWS)
    close(got.float(), want + b.double(), tol, "shared rows with bias")


@pytest.mark.parametrize("M,F,K", [(17, 48, 512), (40, 1008, 1024), (64, 8192, 2048)])
def test_linear_swiglu_shared_rows(ops, M, F, K):
    x, wg, wu = rand((M, K), BF16, 54), rand((F, K), BF16, 55, 0.2), rand((F, K), BF16, 56, 0.2)
    w = ops.interleave_gate_up(wg.to(DEV), wu.to(DEV))
    g, u = x.double() @ wg.double().T, x.double() @ wu.double().T
    want = g / (1 + torch.exp(-g)) * u
    got = ops.linear_swiglu(x.to(DEV), w, force_kernel=SHARED_ROWS)
    close(got.float(), want, BF16_ULP, "shared rows")


@pytest.mark.parametrize("M,N,K,S", [(24, 2048, 8192, 8), (64, 100, 3072, 3), (33, 2048, 2048, 2)])
def test_linear_shared_rows_split_k(ops, M, N, K, S):
    x, w, b = rand((M, K), BF16, 57), rand((N, K), BF16, 58, 0.05), rand((N,), F32, 59)
    parts = ops.linear(x.to(DEV), w.to(DEV), b.to(DEV), partial_sums=True, split_k=S,
                       force_kernel=SHARED_ROWS)
    assert parts.shape == (S, M, N) and parts.dtype == F32
    close(parts.sum(0), x.double() @ w.double().T + b.double(), 2e-5, "sum of the partial sums")


ROWS32 = 12           # force_kernel: 25 to 128 rows (it takes 1 to 128), 32 x 32 tiles, rows via LDS


@pytest.mark.parametrize("M", [1, 31, 65, 96, 97, 128])
@pytest.mark.parametrize("N,K", [(64, 256), (208, 1024), (2048, 2048), (8208, 1536)])
@pytest.mark.parametrize("out_dtype", [F32, BF16])
def test_linear_rows32(ops, M, N, K, out_dtype):
    """The kernel for 25 to 128 rows: every row-tile count, matrices that end inside a block's 64
    columns or inside a wave's 32 (208 = 6 tiles and a half), one and several runs of K, a row
    stride, bias; the matrix in fragment order only, and beside its rows."""
    wide = rand((M, K + 8), BF16, 151)
    x, w, b = wide[:, :K], rand((N, K), BF16, 152), rand((N,), F32, 153)
    want = x.double() @ w.double().T
    tol = 2e-5 if out_dtype == F32 else BF16_ULP
    xd, wd = wide.to(DEV)[:, :K], w.to(DEV)
    kept = ops.InFragments.of(wd)
    got = ops.linear(xd, kept, out_dtype=out_dtype, force_kernel=ROWS32)
    close(got.float(), want, tol, "rows32")
    got = ops.linear(xd, wd, b.to(DEV), out_dtype=out_dtype, force_kernel=ROWS32,
                     weight_frag=ops.fragment_order(wd))
    close(got.float(), want + b.double(), tol, "rows32 with bias")


@pytest.mark.parametrize("M,F,K", [(65, 48, 256), (100, 1008, 1024), (128, 8192, 2048)])
def test_linear_swiglu_rows32(ops, M, F, K):
    x, wg, wu = rand((M, K), BF16, 154), rand((F, K), BF16, 155, 0.2), rand((F, K), BF16, 156, 0.2)
    w = ops.InFragments.of(ops.interleave_gate_up(wg.to(DEV), wu.to(DEV)))
    g, u = x.double() @ wg.double().T, x.double() @ wu.double().T
    want = g / (1 + torch.exp(-g)) * u
    got = ops.linear_swiglu(x.to(DEV), w, force_kernel=ROWS32)
    close(got.float(), want, BF16_ULP, "rows32")
    if M > 24:          # and it is what such a step takes by itself: the same bits
        assert torch.equal(ops.linear_swiglu(x.to(DEV), w), got)


@pytest.mark.parametrize("M,N,K,S", [(128, 2048, 8192, 8), (70, 112, 3072, 3), (99, 2048, 2048, 2),
                                     (128, 6144, 2048, 1)])
def test_linear_rows32_split_k(ops, M, N, K, S):
    x, w, b = rand((M, K), BF16, 157), rand((N, K), BF16, 158, 0.05), rand((N,), F32, 159)
    kept = ops.InFragments.of(w.to(DEV))
    parts = ops.linear(x.to(DEV), kept, b.to(DEV), partial_sums=True, split_k=S,
                       force_kernel=ROWS32)
    want = x.double() @ w.double().T + b.double()
    if S == 1:
        assert parts.shape == (M, N)
        close(parts.float(), want, BF16_ULP, "one range")
        return
    assert parts.shape == (S, M, N) and parts.dtype == F32
    close(parts.sum(0), want, 2e-5, "sum of the partial sums")


def test_linear_rows32_is_what_steps_of_25_to_128_rows_take(ops):
    """Without a kernel asked for, a product of 25 to 128 rows over a matrix in fragment order is
    this kernel's (bit for bit), with the K ranges that the rule gives it; a matrix kept as rows
    only, or a K that is no multiple of 256, goes to the block kernels as before."""
    x, w = rand((100, 2048), BF16, 160).to(DEV), rand((3072, 2048), BF16, 161, 0.05).to(DEV)
    kept = ops.InFragments.of(w)
    assert torch.equal(ops.linear(x, kept), ops.linear(x, kept, force_kernel=ROWS32))
    assert ops.split_k_for(100, 3072, 2048) == 4 and ops.split_k_for(100, 6144, 2048) == 2
    assert ops.split_k_for(128, 2048, 8192) == 8 and ops.split_k_for(65, 16384, 2048) == 1
    assert ops.split_k_for(64, 1024, 4608) == 6          # (not only powers of two)
    parts = ops.linear(x, kept, partial_sums=True)
    assert parts.shape == (4, 100, 3072)
    assert torch.equal(parts, ops.linear(x, kept, partial_sums=True, force_kernel=ROWS32))
    close(ops.linear(x, w).float(), x.double().cpu() @ w.double().cpu().T, BF16_ULP, "rows only")
    with pytest.raises(RuntimeError):
        ops.linear(x, w, force_kernel=ROWS32)                 # no fragment order
    x3, w3 = x[:, :1920].contiguous(), ops.InFragments.of(w[:, :1920].contiguous())
    with pytest.raises(RuntimeError):
        ops.linear(x3, w3, force_kernel=ROWS32)               # 1920 is no multiple of 256
    close(ops.linear(x3, w3).float(), x3.double().cpu() @ w[:, :1920].double().cpu().T, BF16_ULP,
          "K = 1920")


def test_linear_shared_rows_refuses_what_does_not_fit(ops):
    x, w = rand((32, 520), BF16, 60).to(DEV), rand((64, 520), BF16, 61).to(DEV)
    with pytest.raises(RuntimeError):
        ops.linear(x, w, force_kernel=SHARED_ROWS)          # K is no multiple of 512
    with pytest.raises(RuntimeError):
        ops.linear(x[:8, :512].contiguous(), w[:, :512].contiguous(), force_kernel=SHARED_ROWS)


def test_linear_block256_split_k(ops):
    """Partial sums over K ranges from the large-product kernel add up to the product."""
    M, N, K = 2048, 2048, 8192
    x, w = rand((M, K), BF16, 47), rand((N, K), BF16, 48, 0.05)
    S = ops.split_k_for(M, N, K)
    assert S > 1
    parts = ops.linear(x.to(DEV), w.to(DEV), partial_sums=True)
    assert parts.shape == (S, M, N) and parts.dtype == F32
    close(parts.sum(0), x.double() @ w.double().T, 2e-5, "sum of the partial sums")


@pytest.mark.parametrize("M", [1, 3, 8, 16, 40, 200])
@pytest.mark.parametrize("N,K", [(16, 32), (48, 96), (2048, 2048), (1008, 4128), (6144, 1024)])
def test_products_read_the_fragment_order_copy(ops, M, N, K):
    """With the copy of the matrix in fragment order beside it every product gives bit for bit
    what it gives without: plain, with bias, as partial sums over K ranges, with the SwiGLU
    epilogue, adding into the residual stream, on scaled rows, and as the fused conv step (the kernel for 1 to
    16 rows reads the copy; with more rows it is passed and not read)."""
    x = rand((M, K), BF16, 60).to(DEV)
    w, b = rand((N, K), BF16, 61, 0.1).to(DEV), rand((N,), F32, 62).to(DEV)
    wf = ops.fragment_order(w)
    assert wf is not None and wf.shape == w.shape and not torch.equal(wf, w)
    # the copy holds element (n, k) at its place in the piece of 16 rows x 32 of K
    n, k = N - 3, K - 5
    at = ((n // 16) * (K // 32) + k // 32) * 512 + ((k % 32) // 8 * 16 + n % 16) * 8 + k % 8
    assert wf.reshape(-1)[at] == w[n, k]
    # (25 to 128 rows and a K of whole runs of 256: with the copy there the product is another
    # kernel's, which exists for the fragment order only and adds in another order)
    other_kernel = 24 < M <= 128 and K % 256 == 0

    def same(a, c, tol):
        if other_kernel:
            close(a.float(), c.double(), tol, "with the copy")
        else:
            assert torch.equal(a, c)
    for bias in (None, b):
        for out_dtype in (BF16, F32):
            same(ops.linear(x, w, bias, out_dtype=out_dtype, weight_frag=wf),
                 ops.linear(x, w, bias, out_dtype=out_dtype), BF16_ULP if out_dtype == BF16 else 2e-5)
    if K % 64 == 0 and not (other_kernel and K % 512):
        same(ops.linear(x, w, partial_sums=True, split_k=2, weight_frag=wf).sum(0),
             ops.linear(x, w, partial_sums=True, split_k=2).sum(0), 2e-5)
    if N % 32 == 0:
        same(ops.linear_swiglu(x, w, weight_frag=wf), ops.linear_swiglu(x, w), BF16_ULP)
    if 16 < M <= 64 and K % 512 == 0:       # the kernel for 17 to 64 rows reads the copy too
        assert torch.equal(ops.linear(x, w, b, force_kernel=SHARED_ROWS, weight_frag=wf),
                           ops.linear(x, w, b, force_kernel=SHARED_ROWS))
        assert torch.equal(
            ops.linear(x, w, partial_sums=True, split_k=2, force_kernel=SHARED_ROWS, weight_frag=wf),
            ops.linear(x, w, partial_sums=True, split_k=2, force_kernel=SHARED_ROWS))
        if N % 32 == 0:
            assert torch.equal(ops.linear_swiglu(x, w, force_kernel=SHARED_ROWS, weight_frag=wf),
                               ops.linear_swiglu(x, w, force_kernel=SHARED_ROWS))
    if M <= ops.FUSED_MAX_ROWS:
        # the product that adds into the residual stream, and the one that scales its rows
        wn = (1 + rand((N,), F32, 64, 0.1)).to(DEV)
        outs = []
        for frag in (wf, None):
            resid = rand((M, N), F32, 63, 2.0).to(DEV)
            rows = ops.linear(x, w, b, weight_frag=frag, add_into=ops.AddInto(resid, wn, 1e-5))
            data = (ops.FragmentRows(rows.data, M, resid).materialize() if rows.fragment
                    else rows.data)             # (the row slots beyond M hold nothing)
            outs.append((resid, data, rows.ss[:, :M]))
        assert all(torch.equal(a, c) for a, c in zip(*outs))
        if N == K:
            rows = ops.linear(x, w, b, add_into=ops.AddInto(rand((M, N), F32, 63, 2.0).to(DEV), wn,
                                                            1e-5))
            assert torch.equal(ops.linear(rows, w, b, out_dtype=F32, weight_frag=wf),
                               ops.linear(rows, w, b, out_dtype=F32))
    if N % 48 == 0 and M <= 64:
        D, L = N // 3, 3
        taps = rand((D, L), F32, 66, 0.5).to(DEV)
        state = rand((M + 1, D, L - 1), F32, 67).to(DEV)
        pos0 = torch.ones(M, dtype=torch.int32, device=DEV)
        slot = torch.arange(M, dtype=torch.int32, device=DEV)
        outs, states = [], []
        for frag in (wf, None):
            st = state.clone()
            outs.append(ops.linear_shortconv_step(x, w, b, taps, None, st, pos0, slot,
                                                  weight_frag=frag))
            states.append(st)
        assert torch.equal(outs[0], outs[1]) and torch.equal(states[0], states[1])


@pytest.mark.parametrize("M", [1, 8, 16, 24, 40, 64, 65, 200, 300, 1000, 2048])
@pytest.mark.parametrize("N,K", [(16, 32), (48, 96), (2048, 2048), (1008, 4128), (6144, 1024),
                                 (1536, 512), (8192, 256)])
def test_products_read_a_matrix_kept_in_fragment_order_only(ops, M, N, K):
    """A matrix of which only the fragment order is kept (``ops.InFragments``) gives bit for bit
    what its rows give, whatever kernel the row count picks: the kernels for 1 to 16 and 17 to 64
    rows, the block kernel in each of its forms (its loads of W are then pieces of 1 KB), the
    older tile kernel where K is no multiple of 128; plain, with bias, as partial sums, with the
    SwiGLU epilogue."""
    x = rand((M, K), BF16, 160).to(DEV)
    w, b = rand((N, K), BF16, 161, 0.1).to(DEV), rand((N,), F32, 162).to(DEV)
    kept = ops.InFragments.of(w)
    assert kept is not None and kept.shape == w.shape and kept.dtype == BF16
    assert torch.equal(kept.materialize(), w)
    forces = [0]
    if M > 64:
        forces += [3, 4, 5, 6] + ([BLOCK256, BLOCK128, BLOCK128_DEEP, BLOCK192] if K % 128 == 0 else [])
    elif M > 16 and K % 512 == 0:
        forces += [SHARED_ROWS]
    if 24 < M <= 128 and K % 256 == 0:
        # the kernel for 25 to 128 rows exists for the fragment order only: left to itself the
        # product over the kept matrix is that kernel's, over the rows a block kernel's; the two
        # add in another order, so they agree to rounding, not bit for bit
        forces.remove(0)
        close(ops.linear(x, kept, b, out_dtype=F32).float(),
              ops.linear(x, w, b, out_dtype=F32).double(), 2e-5, "another kernel for the kept matrix")
        assert torch.equal(ops.linear(x, kept, b), ops.linear(x, kept, b, force_kernel=ROWS32))
    for force in forces:
        for bias in (None, b):
            for out_dtype in (BF16, F32):
                assert torch.equal(
                    ops.linear(x, kept, bias, out_dtype=out_dtype, force_kernel=force),
                    ops.linear(x, w, bias, out_dtype=out_dtype, force_kernel=force)), (force, out_dtype)
        if K % 256 == 0 and (force != SHARED_ROWS or K % 1024 == 0):
            assert torch.equal(ops.linear(x, kept, partial_sums=True, split_k=2, force_kernel=force),
                               ops.linear(x, w, partial_sums=True, split_k=2, force_kernel=force)), force
        if N % 32 == 0 and force != BLOCK192:
            assert torch.equal(ops.linear_swiglu(x, kept, force_kernel=force),
                               ops.linear_swiglu(x, w, force_kernel=force)), force
    # the first rows of the matrix by themselves (the q rows of a stacked q, k, v)
    if N >= 32:
        first = (N // 32) * 16
        got, want = ops.linear(x, kept.rows(first)), ops.linear(x, w[:first].contiguous())
        if 24 < M <= 128 and K % 256 == 0:     # (two kernels, as above)
            close(got.float(), want.double(), BF16_ULP, "the first rows")
        else:
            assert torch.equal(got, want)
    # rows of it as an embedding table
    ids = torch.tensor([0, N - 1, N // 2, 17 % N, 16 % N], dtype=torch.int32, device=DEV)
    assert torch.equal(ops.embed_rows(ids, kept), ops.embed_rows(ids, w))


def test_a_matrix_kept_in_fragment_order_refuses_what_needs_its_rows(ops):
    w = rand((64, 64), BF16, 163).to(DEV)
    kept = ops.InFragments.of(w)
    assert ops.InFragments.of(w[:40].contiguous()) is None and ops.InFragments.of(w.float()) is None
    with pytest.raises(ValueError, match="second copy"):
        ops.linear(rand((4, 64), BF16, 164).to(DEV), kept, weight_frag=kept.data)
    with pytest.raises(ValueError, match="rows"):
        kept.rows(24)
    # rows of x that are not 16-byte aligned would need the plain kernel, which reads rows of W
    x = rand((4, 72), BF16, 165).to(DEV)[:, 4:68]
    with pytest.raises(ValueError, match="aligned"):
        ops.linear(x, kept)


@pytest.mark.parametrize("M", [1, 2, 5, 8, 13, 16])
@pytest.mark.parametrize("N,K", [(16, 32), (48, 96), (2048, 2048), (1008, 4128), (6144, 1024),
                                 (12288, 4096)])
def test_products_read_rows_in_fragment_order(ops, M, N, K):
    """The norm can write up to 16 rows in the order in which the kernel for 1 to 16 rows loads
    them: the same values at other places, and every product that takes them (plain, with bias,
    partial sums, SwiGLU, the fused conv step, with and without the matrix's fragment-order copy)
    gives bit for bit what it gives from ordinary rows."""
    resid0 = rand((M + 3, K), F32, 70, 2.0).to(DEV)
    wn = (1 + rand((K,), F32, 71, 0.1)).to(DEV)
    w, b = rand((N, K), BF16, 72, 0.1).to(DEV), rand((N,), F32, 73).to(DEV)
    wf = ops.fragment_order(w)
    sel = torch.tensor([(3 * i + 1) % (M + 3) for i in range(M)], dtype=torch.int32, device=DEV)
    for delta, rows in ((None, sel), (rand((M + 3, K), BF16, 74).to(DEV), None),
                        (rand((3, M + 3, K), F32, 75).to(DEV), None)):
        r1, r2 = resid0.clone(), resid0.clone()
        n = M if rows is not None else M + 3
        if n > 16:
            continue
        x = ops.add_rmsnorm(r1, delta, wn, 1e-5, BF16, rows=rows, write_resid=rows is None)
        fr = ops.add_rmsnorm(r2, delta, wn, 1e-5, BF16, rows=rows, write_resid=rows is None,
                             fragment=True)
        assert isinstance(fr, ops.FragmentRows) and fr.shape == x.shape and fr.dtype == BF16
        assert fr.resid_after is r2 and torch.equal(r1, r2)
        assert torch.equal(fr.materialize(), x)
        # element (i, k) lies at its place in the piece of 16 rows x 32 of K
        i, k = n - 1, K - 5
        assert fr.data.reshape(-1)[(k // 32) * 512 + ((k % 32) // 8 * 16 + i) * 8 + k % 8] == x[i, k]
        for frag in (wf, None):
            for bias in (None, b):
                for out_dtype in (BF16, F32):
                    assert torch.equal(
                        ops.linear(fr, w, bias, out_dtype=out_dtype, weight_frag=frag),
                        ops.linear(x, w, bias, out_dtype=out_dtype, weight_frag=frag))
            if K % 64 == 0:
                for S in (2, 4) if K % 128 == 0 else (2,):
                    assert torch.equal(
                        ops.linear(fr, w, partial_sums=True, split_k=S, weight_frag=frag),
                        ops.linear(x, w, partial_sums=True, split_k=S, weight_frag=frag))
            if N % 32 == 0:
                assert torch.equal(ops.linear_swiglu(fr, w, weight_frag=frag),
                                   ops.linear_swiglu(x, w, weight_frag=frag))
            if N % 48 == 0:
                D, L = N // 3, 3
                taps = rand((D, L), F32, 76, 0.5).to(DEV)
                state = rand((n + 1, D, L - 1), F32, 77).to(DEV)
                pos0 = torch.ones(n, dtype=torch.int32, device=DEV)
                slot = torch.arange(n, dtype=torch.int32, device=DEV)
                outs, states = [], []
                for rows_in in (fr, x):
                    st = state.clone()
                    outs.append(ops.linear_shortconv_step(rows_in, w, b, taps, None, st, pos0, slot,
                                                          weight_frag=frag))
                    states.append(st)
                assert torch.equal(outs[0], outs[1]) and torch.equal(states[0], states[1])
        # a product that another kernel is asked for takes the rows as a tensor
        assert torch.equal(ops.linear(fr, w, b, force_kernel=1), ops.linear(x, w, b, force_kernel=1))


def test_rows_in_fragment_order_need_their_sizes(ops):
    wn = torch.ones(64, device=DEV)
    with pytest.raises(ValueError):                                       # 17 rows
        ops.add_rmsnorm(rand((17, 64), F32, 78).to(DEV), None, wn, 1e-5, BF16, fragment=True)
    with pytest.raises(ValueError):                                       # float32 rows
        ops.add_rmsnorm(rand((4, 64), F32, 78).to(DEV), None, wn, 1e-5, F32, fragment=True)
    with pytest.raises(ValueError):                                       # width 40
        ops.add_rmsnorm(rand((4, 40), F32, 78).to(DEV), None, torch.ones(40, device=DEV), 1e-5,
                        BF16, fragment=True)


def test_fragment_order_needs_whole_pieces(ops):
    assert ops.fragment_order(rand((40, 64), BF16, 68)) is None          # rows
    assert ops.fragment_order(rand((48, 72), BF16, 68)) is None          # K
    assert ops.fragment_order(rand((48, 64), F32, 68)) is None
    w = rand((48, 64), BF16, 68).to(DEV)
    x = rand((4, 64), BF16, 69).to(DEV)
    with pytest.raises(ValueError):
        ops.linear(x, w, weight_frag=w[:32])


@pytest.mark.parametrize("M,N,K,S,block", [(575, 1024, 4608, 6, 0), (300, 520, 4096, 2, BLOCK128_DEEP),
                                           (130, 264, 1280, 5, BLOCK128_DEEP),
                                           (1100, 2048, 7168, 7, 0)])
def test_linear_block_split_k_at_prompt_portion_sizes(ops, M, N, K, S, block):
    """Products of a few hundred rows in K ranges of any length that is a multiple of 128 (2 to 16
    tiles a range, odd counts of ranges), in both 128 x 128 forms."""
    x, w, b = rand((M, K), BF16, 49), rand((N, K), BF16, 50, 0.05), rand((N,), F32, 51)
    parts = ops.linear(x.to(DEV), w.to(DEV), b.to(DEV), partial_sums=True, split_k=S,
                       force_kernel=block)
    assert parts.shape == (S, M, N) and parts.dtype == F32
    close(parts.sum(0), x.double() @ w.double().T + b.double(), 2e-5, "sum of the partial sums")
    assert 1 <= ops.split_k_for(M, N, K) <= 8 and K % (128 * ops.split_k_for(M, N, K)) == 0


@pytest.mark.parametrize("M,N,K", [(1, 2048, 2048), (8, 2048, 8192), (16, 96, 1024), (40, 1000, 4096),
                                   (64, 64, 512), (5, 6144, 2048), (64, 2048, 8192), (20, 2048, 2048)])
def test_linear_partial_sums(ops, M, N, K):
    """A decode product split over K: float32 partial sums that add up to the product, and an
    RMSNorm that consumes them like an ordinary residual update."""
    x, w, b = rand((M, K), BF16, 19), rand((N, K), BF16, 20, 0.05), rand((N,), F32, 21)
    want = x.double() @ w.double().T + b.double()
    parts = ops.linear(x.to(DEV), w.to(DEV), b.to(DEV), partial_sums=True)
    S = ops.split_k_for(M, N, K)
    if S == 1:
        assert parts.shape == (M, N) and parts.dtype == BF16
        close(parts.float(), want, BF16_ULP, "unsplit")
        return
    assert parts.shape == (S, M, N) and parts.dtype == F32
    close(parts.sum(0), want, 2e-5, "sum of the partial sums")
    resid = rand((M, N), F32, 22, 2.0)
    wn = 1 + rand((N,), F32, 23, 0.1)
    r_dev = resid.to(DEV).clone()
    got = ops.add_rmsnorm(r_dev, parts, wn.to(DEV), 1e-5, BF16)
    r_ref = resid.clone()
    want_n = ref.add_rmsnorm(r_ref, parts.cpu(), wn, 1e-5, F32)
    close(got.float(), want_n, BF16_ULP, "norm over partial sums")
    close(r_dev, r_ref, 1e-6, "residual")
    rows = torch.tensor([M - 1, 0], dtype=torch.int32)
    got = ops.add_rmsnorm(resid.to(DEV), parts, wn.to(DEV), 1e-5, BF16, rows=rows.to(DEV),
                          write_resid=False)
    close(got.float(), ref.add_rmsnorm(resid.clone(), parts.cpu(), wn, 1e-5, F32, rows=rows,
                                       write_resid=False), BF16_ULP, "selected rows")


def folded_reference(resid, delta, wn, eps, w2, b2):
    """float64: the residual after the sum, and RMSNorm(resid + delta) W2^T + b2."""
    total = resid.double() + delta.double()
    xn = total / torch.sqrt((total * total).mean(dim=1, keepdim=True) + eps) * wn.double()
    y = xn @ w2.double().T
    return total, (y if b2 is None else y + b2.double())


@pytest.mark.parametrize("M", [1, 2, 5, 8, 16])
@pytest.mark.parametrize("N,K,N2", [(48, 64, 80), (2048, 2048, 6144), (200, 520, 304),
                                    (1024, 4096, 64), (2048, 8192, 1000)])
def test_products_fold_the_residual_sum_and_the_norm(ops, M, N, K, N2):
    """Two products of a decode step without a norm kernel between them: the first adds its
    result into the residual stream in place and hands on bf16(resid * norm weight) and the sums
    of squares, the second scales its results by the rows' 1 / rms.  Against float64, with the
    error of one bfloat16 rounding of the rows; and against the two products with the norm
    kernel between them."""
    x = rand((M, K), BF16, 80)
    w1, b1 = rand((N, K), BF16, 81, 0.1), rand((N,), F32, 82)
    wn = 1 + rand((N,), F32, 83, 0.1)
    w2, b2 = rand((N2, N), BF16, 84, 0.1), rand((N2,), F32, 85)
    resid0 = rand((M, N), F32, 86, 2.0)
    delta = x.double() @ w1.double().T + b1.double()
    total, want = folded_reference(resid0, delta, wn, 1e-5, w2, b2)
    for frag in (False, True):
        f1 = ops.fragment_order(w1.to(DEV)) if frag else None
        f2 = ops.fragment_order(w2.to(DEV)) if frag else None
        resid = resid0.to(DEV)
        rows = ops.linear(x.to(DEV), w1.to(DEV), b1.to(DEV), weight_frag=f1,
                          add_into=ops.AddInto(resid, wn.to(DEV), 1e-5))
        assert isinstance(rows, ops.ScaledRows) and rows.resid is resid
        assert rows.fragment == (M >= 8 and N % 32 == 0)
        close(resid, total, 1e-5, "residual after the sum")
        close(rows.ss[:, :M].sum(0), (total * total).sum(1), 1e-5, "sums of squares")
        got = ops.linear(rows, w2.to(DEV), b2.to(DEV), out_dtype=F32, weight_frag=f2)
        close(got, want, 2 * BF16_ULP, "product on scaled rows")
        # what the ordinary norm kernel would have fed the second product with
        xn = ops.add_rmsnorm(resid, None, wn.to(DEV), 1e-5, BF16)
        close(got, ops.linear(xn, w2.to(DEV), b2.to(DEV), out_dtype=F32).cpu().double(),
              2 * BF16_ULP, "against norm kernel + product")
        assert torch.equal(rows.materialize(), xn)
    # without a norm weight the product only adds
    resid = resid0.to(DEV)
    added = ops.linear(x.to(DEV), w1.to(DEV), None, add_into=ops.AddInto(resid))
    assert type(added) is ops.Added
    close(resid, resid0.double() + x.double() @ w1.double().T, 1e-5, "residual after the sum")


@pytest.mark.parametrize("M,F,K", [(1, 8192, 2048), (3, 48, 136), (8, 320, 1024), (16, 64, 2048)])
def test_linear_swiglu_on_scaled_rows(ops, M, F, K):
    x = rand((M, 96), BF16, 87)
    w1, wn = rand((K, 96), BF16, 88, 0.1), 1 + rand((K,), F32, 89, 0.1)
    wg, wu = rand((F, K), BF16, 90, 0.1), rand((F, K), BF16, 91, 0.1)
    w = ops.interleave_gate_up(wg.to(DEV), wu.to(DEV))
    resid = rand((M, K), F32, 92, 2.0).to(DEV)
    rows = ops.linear(x.to(DEV), w1.to(DEV), add_into=ops.AddInto(resid, wn.to(DEV), 1e-5))
    got = ops.linear_swiglu(rows, w, weight_frag=ops.fragment_order(w))
    xn = resid.cpu().double()
    xn = xn / torch.sqrt((xn * xn).mean(dim=1, keepdim=True) + 1e-5) * wn.double()
    g, u = xn @ wg.double().T, xn @ wu.double().T
    close(got.float(), g / (1 + torch.exp(-g)) * u, 3 * BF16_ULP, "swiglu on scaled rows")


@pytest.mark.parametrize("M", [1, 8, 11, 16])
def test_epilogues_write_rows_in_fragment_order(ops, M):
    """With 8 to 16 rows the SwiGLU product and the fused conv step can hand their result to the
    next product in the order in which it loads rows: the same numbers, bit for bit, and the
    next product gives the same result from either."""
    K, F, D, L = 256, 320, 96, 3
    x = rand((M, K), BF16, 110).to(DEV)
    w = ops.interleave_gate_up(rand((F, K), BF16, 111, 0.1).to(DEV), rand((F, K), BF16, 112, 0.1).to(DEV))
    plain, frag = ops.linear_swiglu(x, w), ops.linear_swiglu(x, w, out_fragment=True)
    w2 = rand((48, F), BF16, 113, 0.1).to(DEV)
    if M >= 8:
        assert isinstance(frag, ops.FragmentRows) and frag.shape == (M, F)
        assert torch.equal(frag.materialize(), plain)
        assert torch.equal(ops.linear(frag, w2, out_dtype=F32), ops.linear(plain, w2, out_dtype=F32))
    else:
        assert torch.equal(frag, plain)
    wi = rand((3 * D, K), BF16, 114, 0.2).to(DEV)
    taps = rand((D, L), F32, 115, 0.5).to(DEV)
    state = rand((M + 1, D, L - 1), F32, 116).to(DEV)
    pos0 = torch.full((M,), 3, dtype=torch.int32, device=DEV)
    slot = torch.arange(M, dtype=torch.int32, device=DEV)
    st_a, st_b = state.clone(), state.clone()
    plain = ops.linear_shortconv_step(x, wi, None, taps, None, st_a, pos0, slot)
    frag = ops.linear_shortconv_step(x, wi, None, taps, None, st_b, pos0, slot, out_fragment=True)
    assert torch.equal(st_a, st_b)
    if M >= 8:
        assert torch.equal(frag.materialize(), plain)
    else:
        assert torch.equal(frag, plain)


def test_products_that_cannot_fold_go_the_ordinary_way(ops):
    """More than 16 rows, or a float32 matrix: ``add_into`` is not taken up and the product
    comes back as always; scaled rows that meet a float32 matrix are made by the norm kernel."""
    x, w = rand((20, 64), BF16, 93).to(DEV), rand((32, 64), BF16, 94, 0.1).to(DEV)
    resid = rand((20, 32), F32, 95).to(DEV)
    before = resid.clone()
    out = ops.linear(x, w, add_into=ops.AddInto(resid))
    assert isinstance(out, torch.Tensor) and torch.equal(resid, before)
    out = ops.linear(x[:4].float(), w.float(), add_into=ops.AddInto(resid[:4].contiguous()))
    assert isinstance(out, torch.Tensor) and out.dtype == F32
    wn = (1 + rand((32,), F32, 96, 0.1)).to(DEV)
    r4 = resid[:4].contiguous()
    rows = ops.linear(x[:4], w, add_into=ops.AddInto(r4, wn, 1e-5))
    w32 = rand((24, 32), F32, 97).to(DEV)
    got = ops.linear(rows, w32)
    xn = ref.add_rmsnorm(r4.cpu().clone(), None, wn.cpu(), 1e-5, BF16)
    close(got.float(), xn.double() @ w32.cpu().double().T, BF16_ULP, "product")
    # a width that is no multiple of 8: the product after the folded norm runs in the plain
    # kernel, which scales nothing, so the rows are made by the norm kernel first
    x, w = rand((3, 80), BF16, 98).to(DEV), rand((100, 80), BF16, 99, 0.1).to(DEV)
    wn, r3 = (1 + rand((100,), F32, 100, 0.1)).to(DEV), rand((3, 100), F32, 101, 2.0).to(DEV)
    rows = ops.linear(x, w, add_into=ops.AddInto(r3, wn, 1e-5))
    assert isinstance(rows, ops.ScaledRows)
    w2 = rand((24, 100), BF16, 102, 0.1).to(DEV)
    xn = ref.add_rmsnorm(r3.cpu().clone(), None, wn.cpu(), 1e-5, BF16)
    close(ops.linear(rows, w2, out_dtype=F32), xn.double() @ w2.cpu().double().T, BF16_ULP,
          "product in the plain kernel")


@pytest.mark.parametrize("M,N,K", [(1, 7, 20), (5, 301, 100), (70, 33, 84), (3, 64, 1001)])
@pytest.mark.parametrize("out_dtype", [F32, BF16])
def test_linear_bfloat16_at_widths_that_are_no_multiple_of_8(ops, M, N, K, out_dtype):
    x, w, b = rand((M, K), BF16, 94), rand((N, K), BF16, 95), rand((N,), F32, 96)
    want = x.double() @ w.double().T
    tol = 2e-5 if out_dtype == F32 else BF16_ULP
    got = ops.linear(x.to(DEV), w.to(DEV), out_dtype=out_dtype)
    assert got.dtype == out_dtype
    close(got.float(), want, tol, "plain kernel")
    got = ops.linear(x.to(DEV), w.to(DEV), b.to(DEV), out_dtype=out_dtype, partial_sums=True)
    close(got.float(), want + b.double(), tol, "plain kernel with bias")
    # a row stride that is no multiple of 8 although K is one
    wide = rand((M, 43), BF16, 97).to(DEV)
    w40 = rand((N, 40), BF16, 98)
    got = ops.linear(wide[:, :40], w40.to(DEV), out_dtype=out_dtype)
    close(got.float(), wide[:, :40].cpu().double() @ w40.double().T, tol, "odd row stride")


def test_linear_views_and_mixed_storage(ops):
    # x as the leading columns of a wider buffer (a row stride), as attention hands q over
    wide = rand((20, 96 + 40), BF16, 12).to(DEV)
    w = rand((50, 96), BF16, 13)
    got = ops.linear(wide[:, :96], w.to(DEV))
    close(got.float(), wide[:, :96].cpu().double() @ w.double().T, BF16_ULP, "strided x")
    # a matrix stored in 32 bits is multiplied in 32 bits, whatever the activations are
    w32 = rand((50, 96), F32, 14)
    xb = rand((5, 96), BF16, 15)
    got = ops.linear(xb.to(DEV), w32.to(DEV), out_dtype=F32)
    close(got, xb.double() @ w32.double().T, 3e-6, "float32 matrix, bfloat16 activations")


def test_linear_refuses_what_it_cannot_do(ops):
    with pytest.raises(ValueError, match="multiples of 8"):
        ops.linear(rand((4, 20), BF16, 1).to(DEV), rand((8, 20), BF16, 2).to(DEV), force_kernel=2)
    with pytest.raises(ValueError, match="GPU"):
        ops.linear(rand((4, 16), BF16, 1), rand((8, 16), BF16, 2))


# ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("D", [1, 3, 7, 33, 300, 8, 64, 304, 2048])
@pytest.mark.parametrize("L", [2, 3, 4, 5])
def test_shortconv(ops, dtype, D, L):
    """Segments of 1, 2, 9 and 40 rows, fresh and continued, in two steps so that the state
    written by the first is read by the second (kappai: src/test/test_hybrid.c:78-151)."""
    slots = 6
    taps = rand((D, L), F32, 20, 0.5)
    bias = rand((D,), F32, 21, 0.3)
    state0 = rand((slots, D, L - 1), F32, 22)
    for use_bias in (False, True):
        st_dev, st_ref = state0.to(DEV).clone(), state0.clone()
        for step, (lens, pos0, slot) in enumerate([
                ([1, 2, 9, 40], [0, 5, 0, 17], [3, 0, 5, 1]),
                ([2, 1, 1, 3], [1, 7, 9, 57], [3, 0, 5, 1])]):
            T = sum(lens)
            proj = rand((T, 3 * D), dtype, 23 + step)
            seg_start = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
            row_seg = np.repeat(np.arange(len(lens)), lens).astype(np.int32)
            meta = [torch.from_numpy(a) for a in (row_seg, seg_start, np.asarray(pos0, np.int32),
                                                  np.asarray(slot, np.int32))]
            b = bias if use_bias else None
            got = ops.shortconv(proj.to(DEV), taps.to(DEV), b.to(DEV) if use_bias else None,
                                st_dev, *[m.to(DEV) for m in meta])
            want = ref.shortconv(proj.float(), taps, b, st_ref, *meta)
            close(got.float(), want, BF16_ULP if dtype == BF16 else 2e-6, f"step {step}")
            used = sorted(set(slot))
            close(st_dev[used], st_ref[used], 1e-6, f"state after step {step}")
            untouched = [s for s in range(slots) if s not in used]
            assert torch.equal(st_dev[untouched].cpu(), state0[untouched])


@pytest.mark.parametrize("M,D,K,L,bias", [(1, 64, 64, 3, False), (8, 2048, 2048, 3, False),
                                          (5, 96, 96, 4, True), (33, 48, 120, 2, True),
                                          (64, 320, 72, 5, False), (20, 128, 256, 3, True),
                                          (8, 4096, 512, 3, False), (40, 4112, 64, 3, True)])
def test_linear_shortconv_step(ops, M, D, K, L, bias):
    """The fused decode step of a conv layer against the unfused kernels and the CPU stand-in,
    over two steps so that the state written by the first is read by the second."""
    slots = M + 3
    x = [rand((M, K), BF16, 50 + i) for i in range(2)]
    w = rand((3 * D, K), BF16, 52, 0.2)
    b_in = rand((3 * D,), F32, 53, 0.2) if bias else None
    b_cv = rand((D,), F32, 54, 0.2) if bias else None
    taps = rand((D, L), F32, 55, 0.5)
    state0 = rand((slots, D, L - 1), F32, 56)
    slot = torch.randperm(slots, generator=torch.Generator().manual_seed(3))[:M].to(torch.int32)
    st_f, st_u, st_r = state0.to(DEV).clone(), state0.to(DEV).clone(), state0.clone()
    dev = lambda t: None if t is None else t.to(DEV)
    for step in range(2):
        pos0 = (torch.arange(M, dtype=torch.int32) % 3 if step == 0
                else torch.arange(M, dtype=torch.int32) % 3 + 1)      # some rows start fresh
        fused = ops.linear_shortconv_step(x[step].to(DEV), w.to(DEV), dev(b_in), taps.to(DEV),
                                          dev(b_cv), st_f, pos0.to(DEV), slot.to(DEV))
        proj = ops.linear(x[step].to(DEV), w.to(DEV), dev(b_in))
        seg = torch.arange(M, dtype=torch.int32)
        unfused = ops.shortconv(proj, taps.to(DEV), dev(b_cv), st_u, seg.to(DEV),
                                torch.arange(M + 1, dtype=torch.int32).to(DEV), pos0.to(DEV),
                                slot.to(DEV))
        want = ref.linear_shortconv_step(x[step], w, b_in, taps, b_cv, st_r, pos0, slot)
        close(fused.float(), unfused.float(), BF16_ULP, f"fused against unfused, step {step}")
        close(fused.float(), want.float(), BF16_ULP * 2, f"fused against the stand-in, step {step}")
        close(st_f, st_u, 2 * BF16_ULP, f"state, step {step}")
        close(st_f, st_r, 2e-2, f"state against the stand-in, step {step}")


@pytest.mark.parametrize("D,K,L,bias,frag", [(2048, 2048, 3, False, True), (96, 96, 4, True, True),
                                             (48, 120, 2, True, False), (3072, 1024, 3, False, True),
                                             (4096, 512, 3, False, True)])
@pytest.mark.parametrize("M", [1, 8, 13])
def test_linear_shortconv_step_on_scaled_rows(ops, D, K, L, bias, frag, M):
    """The fused conv step of decoded rows whose RMSNorm is folded into the products around it
    gives what the norm kernel followed by the fused step gives."""
    x0 = rand((M, 64), BF16, 89).to(DEV)
    w0 = rand((K, 64), BF16, 90, 0.2).to(DEV)
    resid = rand((M, K), F32, 90, 2.0).to(DEV)
    wn = (1 + rand((K,), F32, 91, 0.1)).to(DEV)
    w = rand((3 * D, K), BF16, 93, 0.2).to(DEV)
    wf = ops.fragment_order(w) if frag else None
    assert (wf is not None) == (frag and K % 32 == 0)
    b_in = rand((3 * D,), F32, 94, 0.2).to(DEV) if bias else None
    b_cv = rand((D,), F32, 95, 0.2).to(DEV) if bias else None
    taps = rand((D, L), F32, 96, 0.5).to(DEV)
    state0 = rand((M + 2, D, L - 1), F32, 97).to(DEV)
    pos0 = torch.full((M,), 5, dtype=torch.int32, device=DEV)
    slot = torch.arange(1, M + 1, dtype=torch.int32, device=DEV)
    st_a, st_b = state0.clone(), state0.clone()
    rows = ops.linear(x0, w0, add_into=ops.AddInto(resid, wn, 1e-5))
    got = ops.linear_shortconv_step(rows, w, b_in, taps, b_cv, st_a, pos0, slot, weight_frag=wf)
    x = ops.add_rmsnorm(resid, None, wn, 1e-5, BF16)
    want = ops.linear_shortconv_step(x, w, b_in, taps, b_cv, st_b, pos0, slot, weight_frag=wf)
    close(got.float(), want.float().cpu().double(), 3 * BF16_ULP, "fused step on scaled rows")
    close(st_a, st_b.cpu().double(), 3 * BF16_ULP, "state")


# ---------------------------------------------------------------------------------------
def paged_case(seed, dtype, H, G, d, ps, lens_before, lens_new, n_pages=None, shuffle=True):
    """Requests that already hold ``lens_before`` tokens get ``lens_new`` more.  Returns
    everything both implementations need; pools start as NaN."""
    rng = np.random.default_rng(seed)
    S = len(lens_new)
    total = [a + b for a, b in zip(lens_before, lens_new)]
    blocks = [(t + ps - 1) // ps for t in total]
    n_pages = n_pages or sum(blocks) + 3
    perm = rng.permutation(n_pages) if shuffle else np.arange(n_pages)
    bt = np.full((S, max(blocks)), -1, dtype=np.int32)
    k = 0
    for s in range(S):
        for b in range(blocks[s]):
            bt[s, b] = perm[k]
            k += 1
    T = sum(lens_new)
    row_seg = np.repeat(np.arange(S), lens_new).astype(np.int32)
    row_pos = np.concatenate([np.arange(a, a + b) for a, b in zip(lens_before, lens_new)]).astype(
        np.int32)
    k_pool = torch.full((n_pages, G, ps, d), float("nan"), dtype=dtype)
    v_pool = torch.full((n_pages, G, d, ps), float("nan"), dtype=dtype)     # values transposed
    # history: what earlier steps would have stored
    for s in range(S):
        for p in range(lens_before[s]):
            k_pool[bt[s, p // ps], :, p % ps, :] = rand((G, d), dtype, seed * 1000 + s * 100 + p)
            v_pool[bt[s, p // ps], :, :, p % ps] = rand((G, d), dtype, seed * 2000 + s * 100 + p)
    qkv = rand((T, (H + 2 * G) * d), dtype, seed + 5)
    tiles, base = [], 0
    for s, n in enumerate(lens_new):
        nt = (n + 31) // 32
        tiles += [(s, base + r, min(32, n - r), j | (nt << 16)) for j, r in enumerate(range(0, n, 32))]
        base += n
    return dict(qkv=qkv, k_pool=k_pool, v_pool=v_pool, row_pos=torch.from_numpy(row_pos),
                row_seg=torch.from_numpy(row_seg), bt=torch.from_numpy(bt), T=T,
                q_tiles=torch.tensor(tiles, dtype=torch.int32), max_pos=int(row_pos.max()),
                single=all(n == 1 for n in lens_new))


def rope_tables(n, rot_dim, theta=10000.0):
    half = rot_dim // 2
    freq = np.power(theta, -2.0 * np.arange(half) / rot_dim)
    ang = np.arange(n)[:, None] * freq[None, :]
    return (torch.from_numpy(np.cos(ang).astype(np.float32)),
            torch.from_numpy(np.sin(ang).astype(np.float32)))


ATT_CASES = [
    # H, G, d, page, tokens held, new tokens, rot_dim, mode, norm, window
    (4, 2, 16, 4, [0, 5, 9], [7, 1, 3], 16, 1, True, 0),
    (3, 1, 32, 16, [0, 31, 16], [33, 1, 2], 32, 1, True, 0),
    (6, 3, 48, 16, [100, 0], [1, 70], 48, 1, True, 0),
    (8, 8, 64, 64, [63, 64, 200], [2, 1, 1], 64, 1, False, 0),
    (5, 5, 128, 8, [17], [20], 64, 2, True, 0),          # partial, interleaved rotation
    (2, 1, 256, 16, [3, 40], [5, 1], 0, 0, True, 0),      # no rotation
    (4, 2, 64, 16, [90, 0, 45], [1, 50, 6], 64, 1, True, 24),   # window
    (32, 8, 64, 16, [300], [1], 64, 1, True, 0),
    (8, 2, 64, 16, [0, 1, 31, 32, 33, 500, 63, 64], [1] * 8, 64, 1, True, 0),     # decode rows
    (6, 3, 48, 32, [200, 7, 95], [1, 1, 1], 48, 1, True, 40),                   # decode, window
    (16, 1, 32, 16, [130, 2], [1, 1], 32, 1, False, 0),                         # 16 heads a kv head
    (4, 4, 128, 16, [77, 140], [40, 1], 128, 1, True, 0),
    (8, 2, 64, 16, [0, 300, 31], [130, 70, 1], 64, 1, True, 0),                 # 4 heads a kv head
    (8, 1, 128, 32, [250, 0], [45, 97], 128, 1, True, 0),                       # 8 heads a kv head
    (4, 1, 64, 48, [120, 0, 66], [80, 33, 2], 64, 1, True, 50),                 # window, page 48
    (4, 2, 64, 16, [20000, 9000], [1, 1], 64, 1, True, 0),       # decode over more than 64 key splits
    (8, 2, 64, 16, [12000], [70], 64, 1, True, 0),               # a portion after a long history
    (16, 1, 256, 16, [300, 40], [1, 1], 256, 1, False, 0),      # decode: four waves' results fit LDS
    (8, 4, 128, 32, [5000, 0, 129, 1023, 1024, 77], [1] * 6, 128, 1, True, 0),    # decode, head 128
]


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("case", ATT_CASES)
def test_store_and_attention(ops, dtype, case):
    H, G, d, ps, before, new, rot_dim, mode, norm, window = case
    c = paged_case(7, dtype, H, G, d, ps, before, new)
    qn = (1 + rand((d,), F32, 30, 0.2)) if norm else None
    kn = (1 + rand((d,), F32, 31, 0.2)) if norm else None
    cos, sin = rope_tables(max(a + b for a, b in zip(before, new)) + 1, rot_dim or 2)
    dev = {k: (v.to(DEV) if torch.is_tensor(v) else v) for k, v in c.items()}
    tol = BF16_ULP if dtype == BF16 else 3e-6

    ops.qk_norm_rope_store(dev["qkv"], H, G, d, None if qn is None else qn.to(DEV),
                           None if kn is None else kn.to(DEV), 1e-5, cos.to(DEV), sin.to(DEV),
                           rot_dim, mode, dev["k_pool"], dev["v_pool"], dev["row_pos"],
                           dev["row_seg"], dev["bt"], ps)
    qkv_ref, k_ref, v_ref = c["qkv"].float(), c["k_pool"].float(), c["v_pool"].float()
    ref.qk_norm_rope_store(qkv_ref, H, G, d, qn, kn, 1e-5, cos, sin, rot_dim, mode, k_ref, v_ref,
                           c["row_pos"], c["row_seg"], c["bt"], ps)
    close(dev["qkv"][:, :H * d].float(), qkv_ref[:, :H * d], tol, "q")
    written = ~torch.isnan(k_ref)
    assert torch.equal(written, ~torch.isnan(dev["k_pool"].cpu().float())), "other slots touched"
    close(torch.nan_to_num(dev["k_pool"].float()), torch.nan_to_num(k_ref), tol, "k pages")
    close(torch.nan_to_num(dev["v_pool"].float()), torch.nan_to_num(v_ref), 0.0, "v pages")

    scale = 1.0 / math.sqrt(d)
    # reference attention over the pools the kernel itself wrote (rounded as the run stores them)
    want = ref.paged_attention(dev["qkv"].cpu().float(), H, G, d, dev["k_pool"].cpu().float(),
                               dev["v_pool"].cpu().float(), c["row_pos"], c["row_seg"], c["bt"],
                               ps, scale, window=window)
    kernels = ["rows"]
    if dtype == BF16 and ps % 16 == 0 and d % 16 == 0 and d <= 256:
        kernels += ["prefill"] + (["decode-split", "decode-block"]
                                  if c["single"] and H // G <= 16 else [])
        if d in (64, 128) and (H // G) % 4 == 0:
            kernels += ["prefill-shared"]
    for kernel in kernels:
        got = ops.paged_attention(dev["qkv"], H, G, d, dev["k_pool"], dev["v_pool"],
                                  dev["row_pos"], dev["row_seg"], dev["bt"], ps, scale,
                                  window=window, q_tiles=dev["q_tiles"], single_rows=c["single"],
                                  max_position=c["max_pos"],
                                  kernel=kernel if kernel.startswith("decode") else kernel.split("-")[0],
                                  prefill_variant=2 if kernel == "prefill-shared" else 1)
        close(got.float(), want, tol * 2, f"attention kernel {kernel}")


QK_CASES = [
    # H, G, d, page, tokens held, rotation, norm, window, store
    (8, 2, 64, 16, [0, 1, 31, 32, 33, 500, 63, 64, 127, 128, 4095], True, True, 0, True),
    (32, 8, 64, 16, [300, 4000], True, True, 0, True),
    (8, 4, 128, 32, [5000, 0, 129, 1023, 1024, 77, 63, 64], True, True, 0, True),
    (4, 4, 64, 64, [63, 64, 200], False, True, 0, True),           # no rotation
    (6, 3, 64, 16, [15, 16, 700], True, False, 0, True),           # no norm
    (4, 2, 64, 16, [90, 5, 450], True, True, 24, True),            # window
    (8, 2, 64, 16, [0, 40, 127, 128, 2000], True, True, 0, False),  # q only: keys are stored already
]


@pytest.mark.parametrize("case", QK_CASES)
def test_decode_attention_with_norm_rotation_and_store_inside(ops, case, kernel="decode-split"):
    """The decode kernel given the raw projection (``ops.QkPrologue``) against the kernel that
    normalises, rotates and stores followed by the same decode kernel: the same keys and values
    in the same slots of the pools (nothing else touched), and the same attention, at positions
    at the start of a page, at its end, at the edges of a wave's chunk of keys and far out."""
    H, G, d, ps, before, rotate, norm, window, store = case
    n = len(before)
    c = paged_case(11, BF16, H, G, d, ps, before, [1] * n)
    if not store:        # the layer whose keys are read has stored this step's already
        for s, p in enumerate(before):
            page = c["bt"][s, p // ps]
            c["k_pool"][page, :, p % ps, :] = rand((G, d), BF16, 900 + s)
            c["v_pool"][page, :, :, p % ps] = rand((G, d), BF16, 950 + s)
    qn = (1 + rand((d,), F32, 30, 0.2)).to(DEV) if norm else None
    kn = (1 + rand((d,), F32, 31, 0.2)).to(DEV) if norm else None
    cos, sin = rope_tables(max(before) + 1, d)
    cos, sin = (cos.to(DEV), sin.to(DEV)) if rotate else (None, None)
    dev = {k: (v.to(DEV) if torch.is_tensor(v) else v) for k, v in c.items()}
    scale = 1.0 / math.sqrt(d)
    assert ops.decode_takes_qk(d, ps)
    # the two kernels
    k1, v1 = dev["k_pool"].clone(), dev["v_pool"].clone()
    q = ops.qk_norm_rope_store(dev["qkv"].clone(), H, G, d, qn, kn, 1e-5, cos, sin,
                               d if rotate else 0, 1 if rotate else 0, k1, v1, dev["row_pos"],
                               dev["row_seg"], dev["bt"], ps, store_kv=store)
    want = ops.paged_attention(q, H, G, d, k1, v1, dev["row_pos"], dev["row_seg"], dev["bt"], ps,
                               scale, window=window, single_rows=True, max_position=c["max_pos"],
                               kernel=kernel)
    # the one
    k2, v2 = dev["k_pool"].clone(), dev["v_pool"].clone()
    got = ops.paged_attention(dev["qkv"], H, G, d, k2, v2, dev["row_pos"], dev["row_seg"],
                              dev["bt"], ps, scale, window=window, single_rows=True,
                              max_position=c["max_pos"], kernel=kernel,
                              qk=ops.QkPrologue(qn, kn, 1e-5, cos, sin, store_kv=store))
    nan = lambda t: torch.nan_to_num(t.float().cpu(), nan=-7.0)
    assert torch.equal(torch.isnan(k1.float()).cpu(), torch.isnan(k2.float()).cpu()), "slots"
    assert torch.equal(nan(v1), nan(v2)), "v pages"
    # (the sums of squares are added in another order: a key may differ in its last bit)
    close(nan(k2), nan(k1).double(), BF16_ULP, "k pages")
    close(got.float(), want.float().cpu().double(), 2 * BF16_ULP, "attention")
    if not store:
        assert torch.equal(nan(k2), nan(dev["k_pool"])) and torch.equal(nan(v2), nan(dev["v_pool"]))


@pytest.mark.parametrize("H,G,d,window", [(8, 2, 64, 0), (4, 4, 128, 0), (6, 3, 48, 700)])
def test_lone_rows_beside_portions(ops, H, G, d, window):
    """A step of two prompt portions and three single decoded tokens, two of them over long
    contexts: with the single rows left out of the tile table and run through the decode kernel
    (``lone_rows``) the result is that of the tiled kernel over all rows, and of the plain
    kernel."""
    ps = 16
    before, new = [0, 2100, 40, 1300, 7], [70, 1, 33, 1, 1]
    c = paged_case(13, BF16, H, G, d, ps, before, new)
    qn, kn = (1 + rand((d,), F32, 30, 0.2)).to(DEV), (1 + rand((d,), F32, 31, 0.2)).to(DEV)
    cos, sin = rope_tables(max(a + b for a, b in zip(before, new)) + 1, d)
    dev = {k: (v.to(DEV) if torch.is_tensor(v) else v) for k, v in c.items()}
    q = ops.qk_norm_rope_store(dev["qkv"], H, G, d, qn, kn, 1e-5, cos.to(DEV), sin.to(DEV), d, 1,
                               dev["k_pool"], dev["v_pool"], dev["row_pos"], dev["row_seg"],
                               dev["bt"], ps)
    scale = 1.0 / math.sqrt(d)
    args = (q, H, G, d, dev["k_pool"], dev["v_pool"], dev["row_pos"], dev["row_seg"], dev["bt"], ps,
            scale)
    plain = ops.paged_attention(*args, window=window, kernel="rows")
    tiled = ops.paged_attention(*args, window=window, q_tiles=dev["q_tiles"], kernel="prefill",
                                max_position=c["max_pos"])
    close(tiled.float(), plain.float().cpu().double(), 2 * BF16_ULP, "all rows in tiles")
    lone = torch.tensor([70, 104, 105], dtype=torch.int32)
    tiles = torch.tensor([t for t in c["q_tiles"].tolist() if t[0] in (0, 2)], dtype=torch.int32)
    got = ops.paged_attention(*args, window=window, q_tiles=tiles.to(DEV), kernel="prefill",
                              max_position=c["max_pos"], lone_rows=lone.to(DEV),
                              max_lone_position=2100)
    close(got.float(), plain.float().cpu().double(), 2 * BF16_ULP, "lone rows apart")
    rest = [i for i in range(c["T"]) if i not in (70, 104, 105)]
    assert torch.equal(got[rest].cpu(), tiled[rest].cpu()), "the rows in tiles are not touched"


def test_many_lone_rows_of_mixed_lengths_beside_a_portion(ops):
    """Single decoded tokens over 3,000 to 13,000 keys beside a prompt portion, enough of them for
    the decode kernel to settle the keys per split from the listed rows' own lengths (the rows
    reach it through a list): every row against the plain kernel."""
    H, G, d, ps = 4, 2, 64, 16
    gen = np.random.default_rng(9)
    lens = [32] + [int(x) for x in gen.integers(3000, 13001, 24)]       # tokens held after the step
    new = [32] + [1] * 24
    S = len(lens)
    blocks = [(n + ps - 1) // ps for n in lens]
    n_pages = sum(blocks) + 1
    perm = gen.permutation(n_pages - 1) + 1
    bt = np.zeros((S, max(blocks)), dtype=np.int32)
    k = 0
    for s_ in range(S):
        bt[s_, :blocks[s_]] = perm[k:k + blocks[s_]]
        k += blocks[s_]
    k_pool = rand((n_pages, G, ps, d), BF16, 21).to(DEV)
    v_pool = rand((n_pages, G, d, ps), BF16, 22).to(DEV)
    T = sum(new)
    q = rand((T, H * d), BF16, 23).to(DEV)
    row_seg = torch.tensor(np.repeat(np.arange(S), new), dtype=torch.int32).to(DEV)
    row_pos = torch.tensor(list(range(32)) + [n - 1 for n in lens[1:]], dtype=torch.int32).to(DEV)
    tiles = torch.tensor([[0, 0, 32, 0 | (1 << 16)]], dtype=torch.int32).to(DEV)
    lone = torch.arange(32, T, dtype=torch.int32).to(DEV)
    args = (q, H, G, d, k_pool, v_pool, row_pos, row_seg, torch.from_numpy(bt).to(DEV), ps,
            1.0 / math.sqrt(d))
    plain = ops.paged_attention(*args, kernel="rows")
    got = ops.paged_attention(*args, q_tiles=tiles, kernel="prefill", max_position=max(lens) - 1,
                              lone_rows=lone, max_lone_position=max(lens) - 1)
    close(got.float(), plain.float().cpu().double(), 2 * BF16_ULP, "lone rows of mixed lengths")


def test_decode_attention_refuses_a_prologue_it_cannot_do(ops):
    c = paged_case(12, BF16, 4, 2, 48, 16, [5], [1])
    dev = {k: (v.to(DEV) if torch.is_tensor(v) else v) for k, v in c.items()}
    assert not ops.decode_takes_qk(48, 16) and not ops.decode_takes_qk(256, 16)
    with pytest.raises(ValueError, match="do not take the norm"):
        ops.paged_attention(dev["qkv"], 4, 2, 48, dev["k_pool"], dev["v_pool"], dev["row_pos"],
                            dev["row_seg"], dev["bt"], 16, 0.1, single_rows=True, max_position=5,
                            kernel="decode", qk=ops.QkPrologue(None, None, 1e-5, None, None))


@pytest.mark.parametrize("case", ATT_CASES)
@pytest.mark.parametrize("n_parts", [1, 3])
def test_store_from_partial_sums(ops, case, n_parts):
    """The projection handed over as float partial sums (a product split over its input
    dimension): the same q, keys and values as from their bfloat16 sum."""
    H, G, d, ps, before, new, rot_dim, mode, norm, window = case
    c = paged_case(7, BF16, H, G, d, ps, before, new)
    qn = (1 + rand((d,), F32, 30, 0.2)) if norm else None
    kn = (1 + rand((d,), F32, 31, 0.2)) if norm else None
    cos, sin = rope_tables(max(a + b for a, b in zip(before, new)) + 1, rot_dim or 2)
    T, W = c["qkv"].shape
    parts = rand((n_parts, T, W), F32, 32)
    total = parts[0].clone()
    for i in range(1, n_parts):
        total += parts[i]
    qkv = total.to(BF16)
    dev = {k: (v.to(DEV) if torch.is_tensor(v) else v) for k, v in c.items()}
    args = (H, G, d, None if qn is None else qn.to(DEV), None if kn is None else kn.to(DEV), 1e-5,
            cos.to(DEV), sin.to(DEV), rot_dim, mode)
    k2, v2 = dev["k_pool"].clone(), dev["v_pool"].clone()
    q_parts = ops.qk_norm_rope_store(parts.to(DEV), *args, dev["k_pool"], dev["v_pool"],
                                     dev["row_pos"], dev["row_seg"], dev["bt"], ps)
    q_whole = ops.qk_norm_rope_store(qkv.to(DEV), *args, k2, v2, dev["row_pos"], dev["row_seg"],
                                     dev["bt"], ps)
    assert q_parts.shape == (T, H * d) and q_parts.dtype == BF16
    assert torch.equal(q_parts.cpu(), q_whole[:, :H * d].cpu()), "q"
    nan = lambda t: torch.nan_to_num(t.float().cpu(), nan=-7.0)
    assert torch.equal(nan(dev["k_pool"]), nan(k2)), "k pages"
    assert torch.equal(nan(dev["v_pool"]), nan(v2)), "v pages"
    # and q alone, for a layer that reads another layer's keys
    q_only = ops.qk_norm_rope_store(parts[:, :, :H * d].contiguous().to(DEV), *args, None, None,
                                    dev["row_pos"], dev["row_seg"], dev["bt"], ps, store_kv=False)
    assert torch.equal(q_only.cpu(), q_parts.cpu())


@pytest.mark.parametrize("D,L,bias", [(8, 2, False), (304, 3, True), (2048, 3, False), (33, 5, True)])
@pytest.mark.parametrize("n_parts", [1, 2, 4])
def test_shortconv_step_from_partial_sums(ops, D, L, bias, n_parts):
    """The decode step of the short convolution from float partial sums of the projection: the
    same output and state as from their bfloat16 sum, over two steps."""
    M, slots = 9, 12
    taps, cb = rand((D, L), F32, 70, 0.5), (rand((D,), F32, 71, 0.3) if bias else None)
    state0 = rand((slots, D, L - 1), F32, 72)
    slot = torch.randperm(slots, generator=torch.Generator().manual_seed(4))[:M].to(torch.int32)
    st_p, st_w = state0.to(DEV).clone(), state0.to(DEV).clone()
    seg = torch.arange(M, dtype=torch.int32).to(DEV)
    seg_start = torch.arange(M + 1, dtype=torch.int32).to(DEV)
    dev = lambda t: None if t is None else t.to(DEV)
    for step in range(2):
        pos0 = ((torch.arange(M, dtype=torch.int32) % 3) + step).to(DEV)      # some rows start fresh
        parts = rand((n_parts, M, 3 * D), F32, 73 + step)
        total = parts[0].clone()
        for i in range(1, n_parts):
            total += parts[i]
        got = ops.shortconv(parts.to(DEV), taps.to(DEV), dev(cb), st_p, seg, seg_start, pos0,
                            slot.to(DEV))
        want = ops.shortconv(total.to(BF16).to(DEV), taps.to(DEV), dev(cb), st_w, seg, seg_start,
                             pos0, slot.to(DEV))
        assert got.dtype == BF16 and torch.equal(got.cpu(), want.cpu()), f"step {step}"
        assert torch.equal(st_p.cpu(), st_w.cpu()), f"state after step {step}"


@pytest.mark.parametrize("D,L,bias,n_parts", [(64, 3, False, 2), (2048, 3, False, 4), (100, 4, True, 3),
                                              (48, 2, True, 2), (320, 5, False, 8)])
def test_shortconv_of_prompt_portions_from_partial_sums(ops, D, L, bias, n_parts):
    """Segments of several rows (prompt portions beside single decoded tokens) from float partial
    sums of the projection: the same output and state, bit for bit, as from their bfloat16 sum,
    over two steps, whichever of the conv kernels the sizes pick."""
    slots = 6
    taps, cb = rand((D, L), F32, 170, 0.5), (rand((D,), F32, 171, 0.3) if bias else None)
    state0 = rand((slots, D, L - 1), F32, 172)
    st_p, st_w = state0.to(DEV).clone(), state0.to(DEV).clone()
    dev = lambda t: None if t is None else t.to(DEV)
    for step, (lens, pos0, slot) in enumerate([([1, 2, 9, 70], [0, 5, 0, 17], [3, 0, 5, 1]),
                                               ([2, 1, 1, 3], [1, 7, 9, 87], [3, 0, 5, 1])]):
        T = sum(lens)
        parts = rand((n_parts, T, 3 * D), F32, 173 + step)
        total = parts[0].clone()
        for i in range(1, n_parts):
            total += parts[i]
        seg_start = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        row_seg = np.repeat(np.arange(len(lens)), lens).astype(np.int32)
        meta = [torch.from_numpy(a).to(DEV) for a in (row_seg, seg_start, np.asarray(pos0, np.int32),
                                                      np.asarray(slot, np.int32))]
        got = ops.shortconv(parts.to(DEV), taps.to(DEV), dev(cb), st_p, *meta)
        want = ops.shortconv(total.to(BF16).to(DEV), taps.to(DEV), dev(cb), st_w, *meta)
        assert got.dtype == BF16 and torch.equal(got.cpu(), want.cpu()), f"step {step}"
        assert torch.equal(st_p.cpu(), st_w.cpu()), f"state after step {step}"


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_attention_finds_one_far_key(ops, dtype):
    """Among 700 keys one is made to match the query: the output must be its value.  A kernel
    that skips a key, a page or a tile's edge fails here, wherever the key lies."""
    H, G, d, ps = 4, 2, 64, 16
    n = 700
    for far in (0, 15, 16, 63, 64, 65, 319, 640, 698, 699):
        c = paged_case(11, dtype, H, G, d, ps, [n], [1])
        q = torch.zeros(d)
        q[3] = 40.0
        c["qkv"][0, :H * d] = q.repeat(H).to(dtype)
        c["k_pool"].zero_()
        c["v_pool"].copy_(rand(c["v_pool"].shape, dtype, 12))
        bt = c["bt"]
        c["k_pool"][bt[0, far // ps], :, far % ps, 3] = 8.0
        marker = rand((G, d), dtype, 13) + 3.0
        c["v_pool"][bt[0, far // ps], :, :, far % ps] = marker
        dev = {k: (v.to(DEV) if torch.is_tensor(v) else v) for k, v in c.items()}
        # the query's own key (position n) must exist too: store zeros for it
        dev["k_pool"][bt[0, n // ps], :, n % ps, :] = 0
        want = marker.float().repeat_interleave(H // G, dim=0).reshape(1, H * d)
        for kernel in (["rows", "prefill", "decode-split", "decode-block"] if dtype == BF16
                       else ["rows"]):
            got = ops.paged_attention(dev["qkv"], H, G, d, dev["k_pool"], dev["v_pool"],
                                      dev["row_pos"], dev["row_seg"], dev["bt"], ps,
                                      1.0 / math.sqrt(d), q_tiles=dev["q_tiles"], single_rows=True,
                                      max_position=c["max_pos"], kernel=kernel, prefill_variant=1)
            close(got.float(), want, 2 * BF16_ULP if dtype == BF16 else 1e-5,
                  f"far key at {far}, kernel {kernel}")


@pytest.mark.parametrize("lengths", ["many long rows", "a few long rows", "a window"])
def test_decode_attention_over_many_rows_of_mixed_lengths(ops, lengths):
    """The decode kernel settles the keys per split from the lengths of all the step's rows: more
    rows than a wave has lanes, where the rows' keys together decide (many long rows) and where
    the longest row does (a few long ones among short ones), and with a window.  Every row against
    the plain attention over its own keys; one far key of the longest row is made to stand out."""
    H, G, d, ps = 4, 2, 64, 16
    window = 0
    gen = np.random.default_rng(5)
    if lengths == "many long rows":
        lens = [int(x) for x in gen.integers(2500, 3001, 100)] + [int(x) for x in gen.integers(1, 200, 50)]
    elif lengths == "a few long rows":
        lens = [6000, 5999, 4097] + [int(x) for x in gen.integers(1, 100, 67)]
    else:
        lens, window = [int(x) for x in gen.integers(1, 6000, 150)], 3000
    gen.shuffle(lens)
    T = len(lens)
    blocks = [(n + ps - 1) // ps for n in lens]
    n_pages = sum(blocks) + 1
    perm = gen.permutation(n_pages - 1) + 1
    bt = np.zeros((T, max(blocks)), dtype=np.int32)
    k = 0
    for t in range(T):
        bt[t, :blocks[t]] = perm[k:k + blocks[t]]
        k += blocks[t]
    k_pool = rand((n_pages, G, ps, d), BF16, 21)
    v_pool = rand((n_pages, G, d, ps), BF16, 22)
    qkv = rand((T, (H + 2 * G) * d), BF16, 23)
    # the longest row: its key number 70 matches the query of head 1 and nothing else does
    far_row, far = int(np.argmax(lens)), 70 if not window else max(lens) - window + 5
    qkv[far_row, d:2 * d] = 0
    qkv[far_row, d + 3] = 60.0
    k_pool[torch.from_numpy(bt[far_row, :blocks[far_row]]).long(), 0, :, 3] = 0
    k_pool[bt[far_row, far // ps], 0, far % ps, 3] = 8.0
    row_pos = torch.tensor([n - 1 for n in lens], dtype=torch.int32)
    row_seg = torch.arange(T, dtype=torch.int32)
    scale = 1.0 / math.sqrt(d)
    want = ref.paged_attention(qkv.float(), H, G, d, k_pool.float(), v_pool.float(), row_pos,
                               row_seg, torch.from_numpy(bt), ps, scale, window=window)
    got = ops.paged_attention(qkv.to(DEV), H, G, d, k_pool.to(DEV), v_pool.to(DEV),
                              row_pos.to(DEV), row_seg.to(DEV), torch.from_numpy(bt).to(DEV), ps,
                              scale, window=window, single_rows=True, max_position=max(lens) - 1,
                              kernel="decode-split")
    close(got.float().cpu(), want, 2 * BF16_ULP, f"decode attention, {lengths}")
    marker = v_pool[bt[far_row, far // ps], 0, :, far % ps].float()
    close(got[far_row, d:2 * d].float().cpu(), marker, 2 * BF16_ULP, "the far key's value")


def test_attention_shared_tiles_find_one_far_key(ops):
    """The same for the kernel that shares key tiles between four heads of a kv head: a prompt
    portion of 40 rows after 700 cached keys; every row's query matches one far key only."""
    H, G, d, ps = 8, 2, 64, 16
    n, new = 700, 40
    for far in (0, 15, 16, 31, 32, 63, 64, 65, 319, 640, 698, 699, 700, 731):
        c = paged_case(11, BF16, H, G, d, ps, [n], [new])
        q = torch.zeros(d)
        q[3] = 40.0
        c["qkv"][:, :H * d] = q.repeat(H).to(BF16)
        c["k_pool"].zero_()
        c["v_pool"].copy_(rand(c["v_pool"].shape, BF16, 12))
        bt = c["bt"]
        c["k_pool"][bt[0, far // ps], :, far % ps, 3] = 8.0
        marker = rand((G, d), BF16, 13) + 3.0
        c["v_pool"][bt[0, far // ps], :, :, far % ps] = marker
        # positions past the cached keys are the rows' own: zero keys, random values
        for p in range(n, n + new):
            if p != far:
                c["k_pool"][bt[0, p // ps], :, p % ps, :] = 0
        dev = {k: (v.to(DEV) if torch.is_tensor(v) else v) for k, v in c.items()}
        got = ops.paged_attention(dev["qkv"], H, G, d, dev["k_pool"], dev["v_pool"],
                                  dev["row_pos"], dev["row_seg"], dev["bt"], ps,
                                  1.0 / math.sqrt(d), q_tiles=dev["q_tiles"], kernel="prefill",
                                  prefill_variant=2)
        want = marker.float().repeat_interleave(H // G, dim=0).reshape(1, H * d)
        # rows that can see the far key return its value
        first = max(0, far - n)
        close(got[first:].float(), want.expand(new - first, -1), 2 * BF16_ULP,
              f"far key at {far}")


# ---------------------------------------------------------------------------------------
def test_sample_rows(ops):
    # a vocabulary that is no multiple of 4, one that fills the registers of the block exactly,
    # and one beyond them (the kernel that reads the row again)
    for V in (1003, 65536, 70001):
        logits = rand((6, V), F32, 40, 3.0)
        logits[0, 17] = logits[0, 900] = 50.0          # a tie: the lowest id wins
        logits[1, V - 1] = 60.0
        temp = torch.tensor([0.0, 0.0, 0.8, 0.8, 2.0, 0.3])
        u = torch.tensor([0.5, 0.5, 0.0, 0.999999, 0.37, 0.62])
        got = ops.sample_rows(logits.to(DEV), temp.to(DEV), u.to(DEV)).cpu()
        want = ref.sample_rows(logits, temp, u)
        assert got.tolist() == want.tolist(), V
        assert got[0] == 17 and got[1] == V - 1
    # every place of a small row can be drawn, the last one too
    flat = torch.zeros((1, 7))
    for k in range(7):
        uk = torch.tensor([(k + 0.5) / 7])
        assert int(ops.sample_rows(flat.to(DEV), torch.ones(1).to(DEV), uk.to(DEV))[0]) == k
    assert int(ops.sample_rows(flat.to(DEV), torch.ones(1).to(DEV),
                               torch.tensor([0.99999994]).to(DEV))[0]) == 6
    # many draws follow the distribution
    lg = torch.log(torch.tensor([0.5, 0.2, 0.15, 0.1, 0.03, 0.01, 0.007, 0.003])).repeat(4000, 1)
    uu = torch.rand(4000, generator=torch.Generator().manual_seed(1))
    draws = ops.sample_rows(lg.to(DEV).contiguous(), torch.ones(4000).to(DEV), uu.to(DEV)).cpu()
    freq = torch.bincount(draws.long(), minlength=8).double() / 4000
    assert abs(freq[0] - 0.5) < 0.03 and abs(freq[1] - 0.2) < 0.03


def test_sample_filtered(ops):
    """The candidate-narrowing draw against the plain sampler, row by row: default options,
    top-k only, top-p only, min-p only, ties in the logits, a vocabulary below the cap, and
    vocabularies above the 65,536 values that the kernel keeps in registers."""
    from plain import sampler as plain_sampler
    rng = np.random.default_rng(5)
    for V in (65536, 1003, 300, 70001, 131072):
        n = 12
        logits = (rng.normal(size=(n, V)) * 3).astype(np.float32)
        logits[1, :50] = logits[1, 0]                      # many equal values at the top-k edge
        logits[2] = np.round(logits[2])                    # ties everywhere
        opts = [(0.8, 40, 0.9, 0.1), (1.3, 5, 1.0, 0.0), (0.5, 0, 0.6, 0.0), (1.0, 0, 1.0, 0.3),
                (2.0, 1000, 0.95, 0.01), (0.7, 2, 0.5, 0.5)]
        rows, keep, temp, tp, mp, uni, want = [], [], [], [], [], [], {}
        for r in range(n):
            t, k, p, m = opts[r % len(opts)]
            u = float(np.float32(rng.random()))
            kk = k if 0 < k < V else min(V, 1024)
            rows.append(r); keep.append(kk); temp.append(t); tp.append(p); mp.append(m); uni.append(u)
            want[r] = plain_sampler.sample_filtered(logits[r], t, k, p, m, u)
        out = torch.full((n,), -1, dtype=torch.int32, device=DEV)
        f32 = lambda v: torch.tensor(v, dtype=torch.float32, device=DEV)
        i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
        ops.sample_filtered(torch.from_numpy(logits).to(DEV), i32(rows), i32(keep), f32(temp),
                            f32(tp), f32(mp), f32(uni), out)
        got = out.cpu().tolist()
        for r in range(n):
            if got[r] != want[r]:
                # equal logits may be ordered differently: the pick must then have the same value
                assert logits[r, got[r]] == logits[r, want[r]], (V, r, got[r], want[r])


def test_sampling_kernels_write_a_second_place(ops):
    """Every sampling kernel writes its tokens to ``also`` as well when given (the token table of
    the decode step that is queued next): the same tokens in both places, nothing else of
    ``also`` touched."""
    rng = np.random.default_rng(9)
    for V in (3000, 70001):
        n = 6
        logits = torch.from_numpy((rng.normal(size=(n, V)) * 3).astype(np.float32)).to(DEV)
        temp = torch.tensor([0.0, 0.9, 0.0, 1.2, 0.0, 0.7], device=DEV)
        uni = torch.rand(n, generator=torch.Generator().manual_seed(3)).to(DEV)
        out = torch.full((n,), -1, dtype=torch.int32, device=DEV)
        also = torch.full((n,), -7, dtype=torch.int32, device=DEV)
        ops.sample_rows(logits, temp, uni, out=out, also=also)
        assert torch.equal(out, also) and torch.equal(out, ops.sample_rows(logits, temp, uni))
        rows = torch.tensor([1, 3], dtype=torch.int32, device=DEV)
        args = (rows, torch.tensor([40, 900], dtype=torch.int32, device=DEV), temp[rows.long()],
                torch.tensor([0.9, 0.95], device=DEV), torch.tensor([0.05, 0.0], device=DEV),
                uni[rows.long()])
        before = out.clone()
        ops.sample_filtered(logits, *args, out, also=also)
        assert torch.equal(out, also)
        assert torch.equal(out[[0, 2, 4, 5]], before[[0, 2, 4, 5]])
        wide = (rows, torch.tensor([1500, 2000], dtype=torch.int32, device=DEV)) + args[2:]
        ops.sample_filtered(logits, *wide, out, wide=True, also=also)
        assert torch.equal(out, also) and torch.equal(out[[0, 2, 4, 5]], before[[0, 2, 4, 5]])


def test_sample_filtered_with_a_top_k_above_what_lds_holds(ops):
    """A top-k above 1024 (the kernel that sorts the whole row in a workspace) against the plain
    sampler: vocabularies below and above a power of two and above the 4096 values that one pass
    of its sort holds in LDS, top-k just above the other kernel's limit and just below the
    vocabulary, with and without top-p and min-p, ties at the edge of the top-k."""
    from plain import sampler as plain_sampler
    rng = np.random.default_rng(6)
    for V in (1500, 4096, 5000, 65536, 70001):
        opts = [(0.8, 1025, 0.9, 0.1), (1.3, V - 1, 1.0, 0.0), (0.5, 1400, 0.6, 0.0),
                (1.0, V - 3, 1.0, 0.3), (2.0, 1200, 0.999, 0.0), (5.0, V - 1, 0.9999, 0.0)]
        n = len(opts)
        logits = (rng.normal(size=(n, V)) * 3).astype(np.float32)
        logits[0, 1000:1100] = logits[0].max() + 1.0       # equal values across the top-k edge
        logits[2] = np.round(logits[2] * 4) / 4            # ties everywhere
        rows, keep, temp, tp, mp, uni, want = [], [], [], [], [], [], {}
        for r, (t, k, p, m) in enumerate(opts):
            u = float(np.float32(rng.random()))
            rows.append(r); keep.append(k); temp.append(t); tp.append(p); mp.append(m); uni.append(u)
            want[r] = plain_sampler.sample_filtered(logits[r], t, k, p, m, u)
        out = torch.full((n,), -1, dtype=torch.int32, device=DEV)
        f32 = lambda v: torch.tensor(v, dtype=torch.float32, device=DEV)
        i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
        ops.sample_filtered(torch.from_numpy(logits).to(DEV), i32(rows), i32(keep), f32(temp),
                            f32(tp), f32(mp), f32(uni), out, wide=True)
        got = out.cpu().tolist()
        for r in range(n):
            if got[r] != want[r]:
                # equal logits may be ordered differently: the pick must then have the same value
                assert logits[r, got[r]] == logits[r, want[r]], (V, r, got[r], want[r])
    # the two kernels agree where both can run
    V = 3000
    logits = torch.from_numpy((rng.normal(size=(8, V)) * 2).astype(np.float32)).to(DEV)
    args = (torch.arange(8, dtype=torch.int32, device=DEV),
            torch.tensor([1, 2, 40, 64, 65, 500, 1024, 1000], dtype=torch.int32, device=DEV),
            torch.full((8,), 0.9, device=DEV), torch.full((8,), 0.95, device=DEV),
            torch.full((8,), 0.02, device=DEV), torch.rand(8, generator=torch.Generator().manual_seed(2)).to(DEV))
    a = torch.full((8,), -1, dtype=torch.int32, device=DEV)
    b = torch.full((8,), -1, dtype=torch.int32, device=DEV)
    ops.sample_filtered(logits, *args, a)
    ops.sample_filtered(logits, *args, b, wide=True)
    assert a.tolist() == b.tolist()


def test_repeat_penalty(ops):
    logits = torch.tensor([[1.0, 0.9, 0.0, -1.0], [2.0, -2.0, 0.5, 0.0]])
    row_start = torch.tensor([0, 3, 4], dtype=torch.int32)
    toks = torch.tensor([0, 3, 0, 1], dtype=torch.int32)
    pen = torch.tensor([2.0, 1.5])
    dev = logits.to(DEV).clone()
    ops.repeat_penalty(dev, row_start.to(DEV), toks.to(DEV), pen.to(DEV))
    want = logits.clone()
    ref.repeat_penalty(want, row_start, toks, pen)
    assert torch.allclose(dev.cpu(), want)
    assert want[0].tolist() == pytest.approx([0.25, 0.9, 0.0, -2.0])


def test_repeat_penalty_of_long_windows_is_the_walk_over_the_list_bit_for_bit(ops):
    """Windows longer than a wave with tokens that come up many times, tokens out of range and
    rows without a penalty: the kernel's lanes share the list, the result is that of one walk
    over it in order (what the reference does, src/sampler.c:205-216), to the last bit."""
    g = torch.Generator().manual_seed(3)
    V, rows = 1000, 5
    logits = torch.randn(rows, V, generator=g) * 3
    logits[0, 7] = 0.0
    lens = [300, 0, 64, 65, 1]
    toks = torch.cat([torch.randint(0, 40, (n,), generator=g) for n in lens]).to(torch.int32)
    toks[5], toks[17] = -1, V + 3
    row_start = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32)
    pen = torch.tensor([1.3, 2.0, 1.0, 0.7, 1.1])
    dev = logits.to(DEV).clone()
    ops.repeat_penalty(dev, row_start.to(DEV), toks.to(DEV), pen.to(DEV))
    want = logits.clone()
    for r in range(rows):
        if float(pen[r]) == 1.0:
            continue
        for t in toks[int(row_start[r]):int(row_start[r + 1])].tolist():
            if 0 <= t < V:
                v = want[r, t]
                want[r, t] = v / pen[r] if v > 0 else v * pen[r]
    assert torch.equal(dev.cpu(), want)


def test_token_history_on_the_gpu(ops):
    """The rings of recent tokens: written anew for some slots, appended to token by token past
    their capacity, and the repeat penalty over their last n tokens, against the same walk on the
    host (bit for bit): windows shorter and longer than what a ring has seen, a window that
    wraps round the ring's end, a token that comes up many times, a row without a penalty."""
    g = torch.Generator().manual_seed(7)
    cap, slots, V = 32, 5, 200
    hist = torch.full((slots, cap), -7, dtype=torch.int32)
    seen = torch.zeros(slots, dtype=torch.int32)
    dh, ds = hist.to(DEV), seen.to(DEV)
    first = {3: [5, 9, 5, 5, 1], 0: list(range(40, 40 + cap)), 4: [17]}
    sl = torch.tensor(list(first), dtype=torch.int32)
    starts = torch.tensor(np.cumsum([0] + [len(v) for v in first.values()]), dtype=torch.int32)
    toks = torch.tensor([t for v in first.values() for t in v], dtype=torch.int32)
    ops.history_set(dh, ds, sl.to(DEV), starts.to(DEV), toks.to(DEV))
    ref.history_set(hist, seen, sl, starts, toks)
    # 50 steps of three requests (rows 2, 0, 1 of the logits; slots 3, 0, 4)
    rows = torch.tensor([2, 0, 1], dtype=torch.int32)
    use = torch.tensor([3, 0, 4], dtype=torch.int32)
    pen = torch.tensor([1.7, 1.2, 1.0])
    last_n = torch.tensor([6, 64, 3], dtype=torch.int32)
    for step in range(50):
        logits = torch.randn(3, V, generator=g) * 2
        dl = logits.to(DEV).clone()
        ops.repeat_penalty_history(dl, rows.to(DEV), use.to(DEV), pen.to(DEV), last_n.to(DEV), dh, ds)
        ref.repeat_penalty_history(logits, rows, use, pen, last_n, hist, seen)
        assert torch.equal(dl.cpu(), logits), step
        chosen = torch.randint(0, 12, (3,), generator=g, dtype=torch.int32)
        ops.history_append(chosen.to(DEV), rows.to(DEV), use.to(DEV), dh, ds)
        ref.history_append(chosen, rows, use, hist, seen)
    assert torch.equal(dh.cpu(), hist) and torch.equal(ds.cpu(), seen)
    assert seen.tolist() == [cap + 50, 0, 0, 55, 51]
    assert (hist[1] == -7).all() and (hist[2] == -7).all()
