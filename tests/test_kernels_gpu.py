"""Each HIP kernel alone against a plain float64 expression of the same formula,
at sizes other than the tiny models' (odd widths, 8B-shaped rows, long key ranges)."""
import math

import pytest
import torch

import plain
from helpers import rel_err

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.fixture(scope="module")
def kn():
    from longbow_quarrel_amd.kernels.hip import HipKernels

    return HipKernels()


def rnd(shape, seed, dtype=torch.float32, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype).to(DEV)


def i32(values):
    return torch.tensor(list(values), dtype=torch.int32, device=DEV)


# --------------------------------------------------------------------------- rows

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [331, 2048, 2176, 4096, 5000, 8192, 16384, 16392])
def test_embed(kn, dtype, width):
    table = rnd((97, width), 1, dtype)
    toks = i32([5, 96, 0, 5, 33])
    out = torch.empty((5, width), dtype=torch.float32, device=DEV)
    kn.embed(table, toks, out)
    assert torch.equal(out, table[toks.long()].float())
    # an id that is no row of the table (the sampler's "no token", an id past the end) gives zeros
    toks = i32([5, -1, 97, 96, 1 << 30])
    out.fill_(7.0)
    kn.embed(table, toks, out)
    assert torch.equal(out[[0, 3]], table[[5, 96]].float()) and not out[[1, 2, 4]].any()


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,width,eps", [(2, 4096, 1e-5), (7, 331, 3e-6), (1, 64, 1e-6), (3, 5000, 1e-5)])
def test_rmsnorm(kn, out_dtype, rows, width, eps):
    x = rnd((rows, width), 2, scale=5.0)
    w = rnd((width,), 3).abs() * 2
    out = torch.empty((rows, width), dtype=out_dtype, device=DEV)
    kn.rmsnorm(x, w, eps, out)
    want = plain.rms_norm(x.cpu(), w.cpu(), eps)
    assert rel_err(out, want) < (2e-6 if out_dtype == torch.float32 else 5e-3)


@pytest.mark.parametrize("delta_dtype", [torch.float32, torch.bfloat16])
def test_rmsnorm_folds_the_residual_add(kn, delta_dtype):
    x = rnd((5, 777), 4)
    d = rnd((5, 777), 5, delta_dtype)
    w = rnd((777,), 6)
    x0 = x.clone()
    out = torch.empty((5, 777), dtype=torch.float32, device=DEV)
    kn.rmsnorm(x, w, 1e-5, out, delta=d)
    summed = x0.double() + d.double()
    assert rel_err(x, summed) < 1e-6  # the stream itself carries the sum on
    assert rel_err(out, plain.rms_norm(summed.cpu(), w.cpu(), 1e-5)) < 2e-6


def test_add_cast_gather(kn):
    x = rnd((9, 130), 7)
    d = rnd((9, 130), 8, torch.bfloat16)
    x0 = x.clone()
    kn.add(x, d)
    assert torch.equal(x, x0 + d.float())
    b = torch.empty_like(x, dtype=torch.bfloat16)
    kn.cast(x, b)
    assert torch.equal(b, x.to(torch.bfloat16))
    f = torch.empty_like(x)
    kn.cast(b, f)
    assert torch.equal(f, b.float())
    rows = i32([8, 0, 3])
    out = torch.empty((3, 130), dtype=torch.float32, device=DEV)
    kn.gather_rows(x, rows, out)
    assert torch.equal(out, x[rows.long()])
    kn.gather_rows(x, rows, out, delta=d)
    assert torch.equal(out, (x + d.float())[rows.long()])


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_swiglu(kn, out_dtype):
    gu = rnd((6, 2 * 333), 9, scale=3.0)
    out = torch.empty((6, 333), dtype=out_dtype, device=DEV)
    kn.swiglu(gu, out)
    want = plain.swiglu(gu[:, :333].cpu(), gu[:, 333:].cpu())
    assert rel_err(out, want) < (2e-6 if out_dtype == torch.float32 else 5e-3)


# --------------------------------------------------------------------------- linear

@pytest.mark.parametrize("m,n,k", [(1, 64, 64), (5, 331, 80), (70, 130, 333), (129, 65, 17), (3, 1000, 4096),
                                   (16, 4096, 4096), (8, 1000, 14336), (2, 50, 260), (300, 700, 1000), (64, 4096, 520)])
def test_linear_float32(kn, m, n, k):
    x, w = rnd((m, k), 10), rnd((n, k), 11)
    out = torch.empty((m, n), dtype=torch.float32, device=DEV)
    kn.linear(x, w, out)
    want = x.double().cpu() @ w.double().cpu().t()
    assert rel_err(out, want) < 2e-6


@pytest.mark.parametrize("n,k", [(700, 4096), (4100, 1000), (130, 14336), (64, 255)])
def test_linear_float32_gives_a_row_the_same_bits_in_every_launch(kn, n, k):
    """The float32 product has three shapes of launch (up to 16 rows streamed from memory with K shared over a
    block's waves, tiles of 64 x 64, tiles of 128 x 128) and one summation tree: a row comes out bit for bit the
    same alone, among 9, among 40 and among 300 rows, from dense rows and from a view with a stride."""
    x, w = rnd((300, k), 20), rnd((n, k), 21)
    whole = torch.empty((300, n), dtype=torch.float32, device=DEV)
    kn.linear(x, w, whole)
    assert rel_err(whole, x.double().cpu() @ w.double().cpu().t()) < 2e-6
    for rows in (1, 9, 16, 17, 40, 64, 65):
        part = torch.empty((rows, n), dtype=torch.float32, device=DEV)
        kn.linear(x[:rows], w, part)
        assert torch.equal(part, whole[:rows]), rows
    wide = torch.zeros((9, k + 4), dtype=torch.float32, device=DEV)  # rows 16 bytes further apart than they are long
    wide[:, :k] = x[100:109]
    part = torch.empty((9, n), dtype=torch.float32, device=DEV)
    kn.linear(wide[:, :k], w, part)
    assert torch.equal(part, whole[100:109])
    if k % 4 == 0:
        odd = torch.zeros((9, k + 1), dtype=torch.float32, device=DEV)  # rows that do not start at 16-byte addresses
        odd[:, :k] = x[100:109]
        kn.linear(odd[:, :k], w, part)
        assert torch.equal(part, whole[100:109])


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("m,n,k", [
    (1, 4096, 4096), (8, 6144, 4096), (16, 1000, 14336), (3, 40, 72), (13, 17, 8),       # skinny
    (5, 2056, 520), (16, 4104, 14336), (8, 128256, 4096), (2, 2048, 8200),                 # skinny, balanced runs
    (17, 256, 128), (32, 4096, 4096), (33, 515, 1000), (64, 130, 264), (64, 4096, 14336),  # skinny, more row tiles
    (65, 256, 128), (100, 300, 1000), (128, 128, 64), (257, 515, 4096),                   # tiled
    (2048, 1024, 512),
    (40, 2048, 512), (48, 2064, 1024), (64, 6144, 4096), (33, 28672, 512),                 # pipelined, 64-row tiles
    (65, 2048, 512), (128, 4104, 1088), (100, 28672, 512),                                 # pipelined, 128-row tiles
    (129, 3000, 2048), (256, 2048, 4096), (200, 28672, 512),                               # pipelined, 256 x 128 / 64
    (50, 12800, 512), (100, 12800, 512), (200, 12800, 512),                                # their 64-column siblings
    (1000, 12700, 192), (300, 49000, 64), (2048, 6144, 4096),     # pipelined, 256 x 256 tiles
    (1000, 8200, 96), (130, 66000, 32), (2048, 4096, 4000),        # pipelined, 128 x 256 tiles
    (2400, 6144, 128), (3100, 7168, 64),   # more than 8 row tiles: an XCD walks windows of 8 x 4 tiles
    (2048, 28672, 128),                    # 3.5 rounds of tiles: the last half round as 128-column tiles
    (2048, 6144, 192), (300, 6200, 128),   # 256 x 192 tiles, with an edge
])
def test_linear_bfloat16_matrix_cores(kn, out_dtype, m, n, k):
    x, w = rnd((m, k), 12, torch.bfloat16), rnd((n, k), 13, torch.bfloat16)
    out = torch.empty((m, n), dtype=out_dtype, device=DEV)
    kn.linear(x, w, out)
    want = x.double().cpu() @ w.double().cpu().t()
    # float32 accumulation of exact bfloat16 products: only the output rounding is bfloat16-sized
    assert rel_err(out, want) < (1e-5 if out_dtype == torch.float32 else 5e-3)


@pytest.mark.parametrize("m,n,k", [(64, 4096, 4096), (17, 4096, 14336), (40, 2560, 2056), (33, 6144, 4096),
                                   (300, 4096, 4096), (2048, 4096, 14336), (65, 1000, 2048), (130, 4096, 14336),
                                   (256, 2100, 1024), (50, 2100, 1024)])  # (the last: 64-column tiles with an edge)
def test_linear_in_pieces_and_their_consumers(kn, m, n, k):
    """Few columns and several row tiles: K is shared out over blocks and the product comes as
    pieces; the norm, the add and the row gather that take such a delta add the pieces up."""
    pieces = kn.linear_pieces(torch.bfloat16, m, n, k)
    assert pieces > 1
    assert kn.linear_pieces(torch.bfloat16, 8, 4096, k) == 1 and kn.linear_pieces(torch.float32, m, n, k) == 1
    x, w = rnd((m, k), 40, torch.bfloat16), rnd((n, k), 41, torch.bfloat16)
    out = torch.full((pieces, m, n), float("nan"), dtype=torch.float32, device=DEV)
    kn.linear(x, w, out)
    want = x.double().cpu() @ w.double().cpu().t()
    assert rel_err(out.double().sum(0), want) < 1e-5
    whole = torch.empty((m, n), dtype=torch.float32, device=DEV)
    kn.linear(x, w, whole)
    assert rel_err(whole, want) < 1e-5
    from longbow_quarrel_amd.kernels.hip import KernelLibraryError

    with pytest.raises(KernelLibraryError):
        kn.linear(x, w, torch.empty((pieces + 1, m, n), dtype=torch.float32, device=DEV))

    # the consumers' own work: the stream plus the exact sum of the pieces as they are
    res = rnd((m, n), 42)
    summed = res.double().cpu() + out.double().sum(0).cpu()
    r1, normed = res.clone(), torch.empty((m, n), dtype=torch.bfloat16, device=DEV)
    nw = rnd((n,), 43)
    kn.rmsnorm(r1, nw, 1e-5, normed, delta=out)
    assert rel_err(r1, summed) < 1e-6
    assert rel_err(normed, plain.rms_norm(summed, nw.cpu(), 1e-5)) < 5e-3
    r2 = res.clone()
    kn.add(r2, out)
    assert rel_err(r2, summed) < 1e-6
    rows = i32([m - 1, 0, 5])
    picked = torch.empty((3, n), dtype=torch.float32, device=DEV)
    kn.gather_rows(res, rows, picked, delta=out)
    assert rel_err(picked, summed[rows.long().cpu()]) < 1e-6


@pytest.mark.parametrize("m", [1, 8, 12, 16])
@pytest.mark.parametrize("n,k,n2", [(4096, 4096, 6144), (4096, 14336, 28672), (2056, 520, 2304)])
def test_products_around_a_norm(kn, m, n, k, n2):
    """x += act . w^T with the rows' sums of squares left in parts and x * gain in bfloat16, then
    rmsnorm(x) . w2^T as that times w2 with every output row divided by the root mean square:
    against the add, the norm and the products one by one.  Taken up to 16 rows, and up to 12 where the
    pipelined tiles take over from 13 (K in 64s)."""
    parts = kn.linear_fused_parts(torch.bfloat16, m, n, k)
    most = 12 if k % 64 == 0 else 16
    assert kn.linear_fused_parts(torch.bfloat16, most, n, k) > 0 and kn.linear_fused_parts(torch.bfloat16, most + 1, n, k) == 0
    if m > most:
        assert parts == 0
        return
    act, w = rnd((m, k), 50, torch.bfloat16), rnd((n, k), 51, torch.bfloat16, 0.05)
    gain, eps = rnd((n,), 53) + 1.0, 1e-5
    x0 = rnd((m, n), 52)
    x = x0.clone()
    sq = torch.full((m, parts), float("nan"), dtype=torch.float32, device=DEV)
    xg = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEV)
    kn.linear_residual(act, w, x, sq, gain=gain, scaled=xg)
    want_x = x0.double().cpu() + act.double().cpu() @ w.double().cpu().t()
    assert rel_err(x, want_x) < 1e-5
    assert rel_err(sq.double().sum(1), (x.double() ** 2).sum(1)) < 1e-6  # of the float32 rows as they are
    assert torch.equal(xg, (x * gain).to(torch.bfloat16))
    x1, sq1 = x0.clone(), torch.empty_like(sq)
    kn.linear_residual(act, w, x1, sq1)  # without a gain: the stream and the sums only
    assert torch.equal(x1, x) and torch.equal(sq1, sq)

    assert kn.linear_fused_parts(torch.bfloat16, m, n2, n) > 0
    w2 = rnd((n2, n), 54, torch.bfloat16, 0.05)
    xd = x.double().cpu()
    rstd = 1.0 / torch.sqrt((xd * xd).mean(1, keepdim=True) + eps)
    want = (xg.double().cpu() @ w2.double().cpu().t()) * rstd  # with the kernel's own rounding of x * gain
    out32 = torch.empty((m, n2), dtype=torch.float32, device=DEV)
    kn.linear_scaled(xg, sq, eps, w2, out32)
    assert rel_err(out32, want) < 1e-5
    out = torch.empty((m, n2), dtype=torch.bfloat16, device=DEV)
    kn.linear_scaled(xg, sq, eps, w2, out)
    assert rel_err(out, want) < 5e-3
    # against the norm as the plain implementation rounds it (after the division, not before)
    h = plain.round_bf16(plain.rms_norm(xd, gain.double().cpu(), eps))
    assert rel_err(out32, h @ w2.double().cpu().t()) < 5e-3  # two bfloat16 roundings of the same rows
    # the same through the SwiGLU epilogue (gate and up rows interleaved in groups of 8)
    gate, up = w2[: n2 // 2], w2[n2 // 2 :]
    wi = kn.interleave_gate_up(gate.contiguous(), up.contiguous())
    act2 = torch.empty((m, n2 // 2), dtype=torch.bfloat16, device=DEV)
    kn.linear_scaled(xg, sq, eps, wi, act2, swiglu=True)
    assert rel_err(act2, plain.swiglu(want[:, : n2 // 2], want[:, n2 // 2 :])) < 5e-3


def test_a_library_function_called_by_name(kn):
    """What a part with a kernel of its own uses: the function by its name, ctypes arguments, the object's
    stream, the library's error text as an exception."""
    from ctypes import c_int, c_longlong
    from longbow_quarrel_amd.kernels.hip import KernelLibraryError, ptr
    x, d = rnd((5, 77), 90), rnd((5, 77), 91)
    want = x + d
    kn.call("lq_add", ptr(x), ptr(d), c_int(0), c_longlong(x.numel()))
    assert torch.equal(x, want)
    with pytest.raises(KernelLibraryError, match="must be positive"):
        kn.call("lq_add", ptr(x), ptr(d), c_int(0), c_longlong(0))
    with pytest.raises(KernelLibraryError, match="no function lq_no_such_kernel"):
        kn.call("lq_no_such_kernel")


def pack_by_hand(w):
    """The packed order written out with views: 8 rows' slabs of 64 k side by side."""
    n, k = w.shape
    return w.view(n // 8, 8, k // 64, 64).permute(0, 2, 1, 3).contiguous().view(n, k)


@pytest.mark.parametrize("n,k", [(2048, 512), (4096, 4096), (6144, 2048), (4096, 1792), (2056, 1024), (8192, 4160),
                                 (28672, 4096)])
def test_a_packed_weight_gives_every_product_the_bits_of_the_dense_one(kn, n, k):
    """Wide bfloat16 weights may be held with 8 rows' slabs of 64 k side by side.  Every kernel that can meet
    such a weight (the balanced kernel up to 32 rows, the pipelined tiles beyond, whole or in shares of K, with
    and without the SwiGLU epilogue, the pair around a norm) reads it and sums in the order it sums a dense one."""
    bf = torch.bfloat16
    w = rnd((n, k), 31, bf, 0.05)
    pw = kn.pack_weight(w)
    assert getattr(pw, "packed", False) and tuple(pw.shape) == (n, k) and pw.dtype == bf
    assert torch.equal(pw.data, pack_by_hand(w))
    assert kn.pack_weight(pw) is pw
    for m in (1, 8, 16, 17, 32, 33, 48, 64, 65, 128, 200, 256, 257, 512, 700, 1024, 2048):
        x = rnd((m, k), 32 + m, bf)
        pieces = kn.linear_pieces(bf, m, n, k)
        shape = (pieces, m, n) if pieces > 1 else (m, n)
        a = torch.full(shape, 7.0, dtype=torch.float32, device=DEV)
        b = torch.full(shape, 9.0, dtype=torch.float32, device=DEV)
        kn.linear(x, w, a)
        kn.linear(x, pw, b)
        assert torch.equal(a, b), (m, "float32 out", pieces)
        a16 = torch.zeros((m, n), dtype=bf, device=DEV)
        b16 = torch.ones((m, n), dtype=bf, device=DEV)
        kn.linear(x, w, a16)
        kn.linear(x, pw, b16)
        assert torch.equal(a16, b16), (m, "bfloat16 out")
        if n % 16 == 0:
            a16 = torch.zeros((m, n // 2), dtype=bf, device=DEV)
            b16 = torch.ones((m, n // 2), dtype=bf, device=DEV)
            kn.linear_swiglu(x, w, a16)
            kn.linear_swiglu(x, pw, b16)
            assert torch.equal(a16, b16), (m, "swiglu")
        parts = kn.linear_fused_parts(bf, m, n, k)
        if parts > 0:
            gain = 1 + 0.3 * rnd((n,), 33)
            res = []
            for weight in (w, pw):
                stream = rnd((m, n), 34)
                sq = torch.zeros((m, parts), dtype=torch.float32, device=DEV)
                scaled = torch.zeros((m, n), dtype=bf, device=DEV)
                kn.linear_residual(x, weight, stream, sq, gain=gain, scaled=scaled)
                res.append((stream, sq, scaled))
            assert all(torch.equal(p, q) for p, q in zip(*res)), (m, "residual")
            sq_in = rnd((m, 5), 35).abs() * k
            for swiglu in ((False, True) if n % 16 == 0 else (False,)):
                outs = [torch.zeros((m, n // 2 if swiglu else n), dtype=bf, device=DEV) for _ in range(2)]
                kn.linear_scaled(x, sq_in, 1e-5, w, outs[0], swiglu=swiglu)
                kn.linear_scaled(x, sq_in, 1e-5, pw, outs[1], swiglu=swiglu)
                assert torch.equal(outs[0], outs[1]), (m, "scaled", swiglu)
    # a table that is also a head: the embedding reads the packed rows
    toks = i32([5, n - 1, 0, 8, 7, -1, n])
    a = torch.empty((7, k), dtype=torch.float32, device=DEV)
    b = torch.empty((7, k), dtype=torch.float32, device=DEV)
    kn.embed(w, toks, a)
    kn.embed(pw, toks, b)
    assert torch.equal(a, b)


def test_weights_that_no_packed_reader_would_take_stay_dense(kn):
    bf = torch.bfloat16
    for shape, dtype in (((2048, 520), bf), ((2052, 512), bf), ((1024, 4096), bf), ((4096, 448), bf),
                         ((4096, 4096), torch.float32)):
        w = rnd(shape, 36, dtype)
        assert kn.pack_weight(w) is w
    kn.pack_weights = False
    try:
        w = rnd((4096, 4096), 37, bf)
        assert kn.pack_weight(w) is w
    finally:
        kn.pack_weights = True


def test_linear_bfloat16_odd_k_takes_the_generic_kernel(kn):
    x, w = rnd((9, 77), 14, torch.bfloat16), rnd((33, 77), 15, torch.bfloat16)
    out = torch.empty((9, 33), dtype=torch.float32, device=DEV)
    kn.linear(x, w, out)
    assert rel_err(out, x.double().cpu() @ w.double().cpu().t()) < 1e-5


def test_linear_row_does_not_depend_on_the_batch(kn):
    """Row 0 alone (skinny kernel) against row 0 among 300 (tiled kernel): equal up to float32 rounding."""
    x, w = rnd((300, 4096), 16, torch.bfloat16), rnd((512, 4096), 17, torch.bfloat16)
    big = torch.empty((300, 512), dtype=torch.float32, device=DEV)
    one = torch.empty((1, 512), dtype=torch.float32, device=DEV)
    kn.linear(x, w, big)
    kn.linear(x[:1], w, one)
    assert rel_err(one, big[:1]) < 1e-5


# --------------------------------------------------------------------------- rotation + cache write, attention

BS = 64


def paged_cache(lengths, kv_heads, head_dim, dtype, seed, ramp=None):
    """Random keys/values for sequences of the given lengths in a paged cache whose blocks are
    handed out in a shuffled order; returns dense copies too.  With `ramp` the keys' first component is
    ramp(t) at position t."""
    g = torch.Generator().manual_seed(seed)
    need = [(n + BS - 1) // BS for n in lengths]
    n_blocks = sum(need) + 3
    perm = torch.randperm(n_blocks, generator=g).tolist()
    table = torch.zeros((len(lengths) + 2, max(need) + 1), dtype=torch.int32)
    slots = list(range(len(lengths), 0, -1))  # slot ids differ from batch indices
    kc = torch.zeros((n_blocks, kv_heads, BS, head_dim), dtype=dtype)
    vc = torch.zeros((n_blocks, kv_heads, head_dim, BS), dtype=dtype)
    dense = []
    for b, n in enumerate(lengths):
        k = torch.randn((n, kv_heads, head_dim), generator=g)
        if ramp is not None:
            k[:, :, 0] = torch.tensor([ramp(t) for t in range(n)])[:, None]
        k = k.to(dtype)
        v = torch.randn((n, kv_heads, head_dim), generator=g).to(dtype)
        dense.append((k, v))
        for j in range(need[b]):
            blk = perm.pop()
            table[slots[b], j] = blk
            lo, hi = j * BS, min(n, (j + 1) * BS)
            kc[blk, :, : hi - lo, :] = k[lo:hi].transpose(0, 1)
            vc[blk, :, :, : hi - lo] = v[lo:hi].permute(1, 2, 0)
    return kc.to(DEV), vc.to(DEV), table.to(DEV), slots, dense


def run_attention(kn, q_rows, lengths, new, heads, kv_heads, head_dim, dtype, seed, window=0, decode=False,
                  force_generic=False, standout=None, max_len=None, uneven=False, check=None, q_by_position=False,
                  ramp=None):
    """q rows for the last `new[b]` positions of each sequence; returns (got, want).  With `check` (rows of
    the step, counted through all sequences) only these rows are worked out by the plain implementation
    and returned: for steps of thousands of rows.  With `q_by_position` the query of a position of a sequence is
    the same whatever rows the step brings (for comparisons between steps).  With `ramp` the scores of a
    row grow with the key's position by ramp(t) (natural-log units) on top of the random part."""
    kc, vc, table, slots, dense = paged_cache(lengths, kv_heads, head_dim, dtype, seed, ramp)
    g = torch.Generator().manual_seed(seed + 1)
    rows = sum(new)
    q = torch.randn((rows, heads * head_dim), generator=g)
    if ramp is not None:
        q.view(rows, heads, head_dim)[:, :, 0] = math.sqrt(head_dim)  # times the scale: 1
    q = q.to(dtype)
    if q_by_position:
        per_seq = [torch.randn((n, heads * head_dim), generator=torch.Generator().manual_seed(seed + 7 + b)).to(dtype)
                   for b, n in enumerate(lengths)]
        q = torch.cat([qs[n - m:] for qs, n, m in zip(per_seq, lengths, new)])
    if standout is not None:
        # one far key that every query must find: its score stands out by construction
        b, t = standout
        k, v = dense[b]
        k[t] = k[t] * 0 + 1.0
        v[t] = v[t] * 0 + 7.0
        blk = int(table[slots[b], t // BS])
        kc[blk, :, t % BS, :] = 1.0
        vc[blk, :, :, t % BS] = 7.0
        q = q * 0.01 + 3.0
        q = q.to(dtype)
    row_seq, row_pos, cu = [], [], [0]
    for b, (n, m) in enumerate(zip(lengths, new)):
        row_seq += [b] * m
        row_pos += list(range(n - m, n))
        cu.append(cu[-1] + m)
    qd = q.to(DEV)
    out = torch.empty_like(qd)
    scale = 1.0 / math.sqrt(head_dim)
    kn.force_generic = force_generic
    max_len = max_len or max(lengths)
    try:
        need = kn.attention_workspace(dtype, rows, heads, kv_heads, head_dim, BS, decode, max_len)
        ws = torch.empty(need, dtype=torch.float32, device=DEV) if need else None
        kn.attention(qd, out, heads, kv_heads, head_dim, i32(row_pos), i32(row_seq), i32(slots), i32(cu),
                     table, kc, vc, BS, scale, window, decode=decode, max_len=max_len, workspace=ws, uneven=uneven)
    finally:
        kn.force_generic = False
    want = torch.zeros((rows, heads, head_dim), dtype=torch.float64)
    r = 0
    for b, (n, m) in enumerate(zip(lengths, new)):
        k, v = dense[b]
        # plain attention over the whole sequence with the real queries in the last m places
        qfull = torch.zeros((n, heads, head_dim), dtype=torch.float64)
        qfull[n - m:] = q[r : r + m].double().view(m, heads, head_dim)
        places = range(n - m, n) if check is None else [n - m + (c - r) for c in check if r <= c < r + m]
        want[r : r + m] = plain.attention(qfull, k, v, window=window, rows=places)[n - m:]
        r += m
    got = out.view(rows, heads, head_dim)
    if check is not None:
        idx = torch.tensor(sorted(check))
        return got[idx.to(DEV)], want[idx]
    return got, want


@pytest.mark.parametrize("dtype,generic", [(torch.float32, True), (torch.bfloat16, True), (torch.bfloat16, False)])
@pytest.mark.parametrize("heads,kv_heads,head_dim", [(4, 2, 64), (3, 1, 32), (6, 3, 48), (8, 8, 128), (2, 1, 96)])
def test_attention_prompts(kn, dtype, generic, heads, kv_heads, head_dim):
    got, want = run_attention(kn, None, [5, 70, 131, 1], [5, 70, 40, 1], heads, kv_heads, head_dim, dtype, 21,
                              force_generic=generic)
    assert rel_err(got, want) < (2e-6 if dtype == torch.float32 else 8e-3)


@pytest.mark.parametrize("heads,kv_heads,head_dim", [(8, 2, 64), (8, 2, 128), (4, 4, 128), (2, 1, 96)])
@pytest.mark.parametrize("shape", ["slow", "steps", "down"])
def test_attention_when_the_largest_score_keeps_moving(kn, heads, kv_heads, head_dim, shape):
    """The running maximum of the prompt kernels follows the scores lazily (it moves when a score stands far
    enough above it).  Scores that creep up by less than that a chunk, that jump by more every few hundred
    keys, and that fall from a large first key all give the plain implementation's result."""
    ramp = {"slow": lambda t: 0.05 * t,                       # 2.3 in the log2 domain every 32 keys
            "steps": lambda t: 9.0 * (t // 200),              # 13 in the log2 domain every 200 keys
            "down": lambda t: 40.0 - 0.03 * t}[shape]
    got, want = run_attention(kn, None, [700, 333, 40], [700, 300, 40], heads, kv_heads, head_dim, torch.bfloat16, 57,
                              ramp=ramp)
    assert rel_err(got, want) < 8e-3
    if (heads, head_dim) == (8, 128):  # a long sequence too
        got, want = run_attention(kn, None, [2650], [2650], heads, kv_heads, head_dim, torch.bfloat16, 58, ramp=ramp,
                                  check=[0, 40, 700, 1999, 2000, 2001, 2649])
        assert rel_err(got, want) < 8e-3


@pytest.mark.parametrize("heads,kv_heads,head_dim,lengths,new,window", [
    (8, 2, 64, [5, 70, 131, 1, 300], [5, 70, 40, 1, 300], 0),   # four heads a kv head, head size 64: 32 x 32 tiles
    (8, 2, 64, [200, 333], [200, 100], 90),                      # and with a window
    (16, 2, 128, [3100], [3100], 0),                             # head size 128: 32 x 32 tiles as well
    (8, 2, 128, [3200], [3200], 1000),
    (8, 2, 96, [100, 3200 * 2 - 100], [100, 3200 * 2 - 100], 0), # two sequences, one short
    (8, 2, 128, [300] * 9, [300] * 9, 0),                        # many short sequences with partial last tiles
    (8, 2, 128, [700, 64, 257], [700, 64, 200], 0),
    (32, 8, 128, [1100, 333], [1100, 300], 0),                   # more workgroups than compute units: a wave a head
    (16, 8, 128, [1500, 77], [1500, 77], 500),                   # ... two heads a kv head, a window
    (8, 2, 192, [700, 64, 257, 1], [700, 64, 200, 1], 0),        # head sizes above 128: 16 x 16 tiles, four heads a kv head
    (8, 2, 192, [333, 200], [100, 200], 90),                     # ... with a window, partial tiles
    (4, 1, 256, [300, 45], [300, 45], 0),
    (3, 3, 128, [700, 77], [700, 77], 0),                        # one head a kv head at head size 128: 16 x 16 tiles
    (6, 3, 96, [700, 77], [650, 77], 100),                       # two heads a kv head
])
def test_attention_prompts_on_both_tile_shapes(kn, heads, kv_heads, head_dim, lengths, new, window):
    """Prompt attention has a kernel with 32 x 32 score tiles (a wave a head, or two that share a cache block's
    keys where the step has few rows) and one with 16 x 16: which one runs depends on the head size, the heads
    a kv head and the rows of the step.  All against the plain implementation."""
    got, want = run_attention(kn, None, lengths, new, heads, kv_heads, head_dim, torch.bfloat16, 77, window=window)
    assert rel_err(got, want) < 8e-3


@pytest.mark.parametrize("dtype,generic", [(torch.float32, True), (torch.bfloat16, False)])
@pytest.mark.parametrize("heads,kv_heads,head_dim", [(32, 8, 128), (3, 1, 32), (16, 1, 64), (6, 3, 48)])
def test_attention_decoding_over_long_keys(kn, dtype, generic, heads, kv_heads, head_dim):
    got, want = run_attention(kn, None, [700, 64, 257, 1, 300], [1, 1, 1, 1, 1], heads, kv_heads, head_dim,
                              dtype, 22, decode=True, force_generic=generic)
    assert rel_err(got, want) < (2e-6 if dtype == torch.float32 else 8e-3)


@pytest.mark.parametrize("dtype,generic", [(torch.float32, True), (torch.bfloat16, True), (torch.bfloat16, False)])
@pytest.mark.parametrize("window", [1, 33, 64, 100])
def test_attention_window_edge(kn, dtype, generic, window):
    got, want = run_attention(kn, None, [150, 40], [150, 3], 4, 2, 64, dtype, 23, window=window, force_generic=generic)
    assert rel_err(got, want) < (2e-6 if dtype == torch.float32 else 8e-3)
    got, want = run_attention(kn, None, [300, 99], [1, 1], 4, 2, 64, dtype, 24, window=window, decode=True,
                              force_generic=generic)
    assert rel_err(got, want) < (2e-6 if dtype == torch.float32 else 8e-3)


@pytest.mark.parametrize("head_dim,heads,kv_heads", [(128, 8, 2), (64, 3, 3), (192, 2, 1)])
@pytest.mark.parametrize("window", [0, 257, 600])
def test_decode_attention_over_several_splits(kn, head_dim, heads, kv_heads, window):
    """Rows whose keys lie in up to six splits of 256 positions, the first of them hidden by the window for
    some rows; a row's splits are added up by whichever of its workgroups comes last, and the counters that
    tell which one that is are left at zero for the next launch (so the same launch again gives the same)."""
    lengths = [1500, 900, 256, 257, 64, 1100]
    got, want = run_attention(kn, None, lengths, [1] * len(lengths), heads, kv_heads, head_dim, torch.bfloat16, 31,
                              window=window, decode=True)
    assert rel_err(got, want) < 8e-3
    again, _ = run_attention(kn, None, lengths, [1] * len(lengths), heads, kv_heads, head_dim, torch.bfloat16, 31,
                             window=window, decode=True)
    assert torch.equal(got, again)
    assert int(kn.tickets(torch.device('cuda', torch.cuda.current_device())).abs().max()) == 0


@pytest.mark.parametrize("rows", [24, 64])
def test_decode_attention_of_many_rows_with_long_splits(kn, rows):
    """24 and 64 sequences of 8 kv heads and head size 128, up to 3 000 keys: so many workgroups that a
    split covers 512 to 3 072 positions (one split for some launches, several for others, with rows of one
    launch ending in different splits).  Twice, with the ticket counters back at zero after each."""
    g = torch.Generator().manual_seed(rows)
    lengths = torch.randint(1, 3001, (rows,), generator=g).tolist()
    lengths[0], lengths[1], lengths[2] = 3000, 1, 1025
    for max_extra in (0, 1100):  # the bound a captured step would pass: lengths rounded up, or a bucket more
        got, want = run_attention(kn, None, lengths, [1] * rows, 32, 8, 128, torch.bfloat16, 61, decode=True,
                                  max_len=max(lengths) + max_extra)
        assert rel_err(got, want) < 8e-3
        for r in (0, 1, 2, rows - 1):  # row by row: a row that a split lost would drown in the whole
            assert rel_err(got[r], want[r]) < 8e-3, (r, lengths[r])
        assert int(kn.tickets(torch.device('cuda', torch.cuda.current_device())).abs().max()) == 0
    again, _ = run_attention(kn, None, lengths, [1] * rows, 32, 8, 128, torch.bfloat16, 61, decode=True,
                             max_len=max(lengths) + 1100)
    assert torch.equal(got, again)


@pytest.mark.parametrize("dtype,generic", [(torch.float32, True), (torch.bfloat16, False)])
@pytest.mark.parametrize("decode", [False, True])
def test_attention_finds_one_far_key_among_hundreds(kn, dtype, generic, decode):
    """Key 3 of 600 carries score ~ 3 * hd / sqrt(hd) above the rest: the output must be its value."""
    new = [1, 1] if decode else [17, 2]
    got, want = run_attention(kn, None, [600, 130], new, 4, 2, 64, dtype, 25, decode=decode, force_generic=generic,
                              standout=(0, 3))
    assert rel_err(got, want) < (2e-6 if dtype == torch.float32 else 8e-3)
    assert float((got[0].double().cpu() - 7.0).abs().max()) < 0.1


def _tickets_are_zero(kn):
    return int(kn.tickets(torch.device('cuda', torch.cuda.current_device())).abs().max()) == 0


@pytest.mark.parametrize("lengths,uneven", [
    ([33000], False),                                       # one sequence: splits that grow beyond 256 keys
    ([131072], False),                                      # the longest context that is quoted anywhere
    ([16384] * 8, False),                                   # a batch of eight at 16 K keys
    ([40000, 300, 2000, 64, 5000, 1, 700, 1500], True),     # one long sequence among short ones, shared out by units
    ([40000, 300, 2000, 64, 5000, 1, 700, 1500], False),    # and as the grid (sequence, kv head, split)
])
def test_decode_attention_at_the_long_contexts_that_are_measured(kn, lengths, uneven):
    """Decoding attention with the 8B shape's heads (32 over 8, head size 128) over 16 K to 128 K keys a
    sequence: block tables of hundreds to thousands of blocks and the split lengths that the launch chooses for
    bounds from 16 K up, against the plain implementation, row by row; twice the same, tickets zero after."""
    n = len(lengths)
    got, want = run_attention(kn, None, lengths, [1] * n, 32, 8, 128, torch.bfloat16, 91, decode=True, uneven=uneven)
    for b in range(n):
        assert rel_err(got[b], want[b]) < 1.2e-2, (b, lengths[b])
    assert rel_err(got, want) < 8e-3
    assert _tickets_are_zero(kn)
    again, _ = run_attention(kn, None, lengths, [1] * n, 32, 8, 128, torch.bfloat16, 91, decode=True, uneven=uneven)
    assert torch.equal(got, again) and _tickets_are_zero(kn)


def test_decode_attention_finds_a_far_key_among_a_hundred_thousand(kn):
    """Key 70 001 of 131 072 stands out by construction (the reference's long-key vectors scaled up:
    internal/device/attention_test.go:10-94): every head's output is its value."""
    got, want = run_attention(kn, None, [131072], [1], 32, 8, 128, torch.bfloat16, 93, decode=True, standout=(0, 70001))
    assert rel_err(got, want) < 8e-3
    assert float((got[0].double().cpu() - 7.0).abs().max()) < 0.1


@pytest.mark.parametrize("lengths,new", [
    ([8192], [8192]),      # a whole prompt of 8 192 rows: the 32 x 32 tiles at head size 128
    ([16384], [8192]),     # the second portion of a 16 384-token prompt: its rows read 8 192 keys that the first left
])
def test_prompt_attention_of_8192_rows(kn, lengths, new):
    """Steps of 8 192 rows at head size 128 (four query heads a kv head), the largest portion that the
    generation loop feeds: rows at the step's start and end, around tile edges and some anywhere, against
    the plain implementation."""
    g = torch.Generator().manual_seed(5)
    check = sorted({0, 1, 31, 32, 33, 63, 64, 255, 256, 4095, 4096, 4097, 8159, 8160, 8190, 8191}
                   | set(torch.randint(0, 8192, (12,), generator=g).tolist()))
    got, want = run_attention(kn, None, lengths, new, 8, 2, 128, torch.bfloat16, 95, check=check)
    for i, row in enumerate(check):
        assert rel_err(got[i], want[i]) < 1.2e-2, row
    assert rel_err(got, want) < 8e-3


@pytest.mark.parametrize("heads,kv_heads", [(64, 8), (16, 2)])
def test_attention_with_eight_query_heads_a_kv_head(kn, heads, kv_heads):
    """The 70B shape's ratio (64 heads over 8 kv heads, head size 128): a decoding step over several splits,
    and prompts on the 16 x 16 tiles (short sequences) and on the 32 x 32 tiles (3 100 rows)."""
    lengths = [1500, 900, 256, 257, 64, 1100, 1, 4200]
    got, want = run_attention(kn, None, lengths, [1] * len(lengths), heads, kv_heads, 128, torch.bfloat16, 97, decode=True)
    assert rel_err(got, want) < 8e-3
    for b in range(len(lengths)):
        assert rel_err(got[b], want[b]) < 1.2e-2, b
    assert _tickets_are_zero(kn)
    got, want = run_attention(kn, None, [300, 64, 257], [300, 64, 100], heads, kv_heads, 128, torch.bfloat16, 98)
    assert rel_err(got, want) < 8e-3
    if heads == 16:
        check = [0, 31, 32, 1000, 3071, 3072, 3098, 3099]
        got, want = run_attention(kn, None, [3100], [3100], heads, kv_heads, 128, torch.bfloat16, 99, check=check)
        assert rel_err(got, want) < 8e-3


@pytest.mark.parametrize("heads,kv_heads,head_dim,window", [(4, 2, 64, 0), (6, 3, 48, 0), (8, 2, 128, 0), (3, 1, 144, 0),
                                                            (4, 2, 16, 0), (4, 4, 32, 70), (5, 1, 20, 0)])
def test_float32_attention_gives_a_row_the_same_bits_in_every_step(kn, heads, kv_heads, head_dim, window):
    """The size-agnostic attention (the whole of the float32 path) works on tiles of 16 rows in prompt steps and
    on single rows in steps of single tokens (head size 20: the kernel with a wavefront a row in both): a row's
    output is the same bits as the last row of a prompt, alone in a decoding step, and in a decoding step among
    other sequences; and right against the plain implementation."""
    lengths = [150, 37, 64, 200]
    whole, want = run_attention(kn, None, lengths, lengths, heads, kv_heads, head_dim, torch.float32, 71, window=window,
                                force_generic=True, q_by_position=True)
    assert rel_err(whole, want) < 2e-6
    last = [sum(lengths[: b + 1]) - 1 for b in range(len(lengths))]
    tail, _ = run_attention(kn, None, lengths, [40, 1, 17, 3], heads, kv_heads, head_dim, torch.float32, 71, window=window,
                            force_generic=True, q_by_position=True)
    ends = [39, 40, 57, 60]
    for b in range(len(lengths)):
        assert torch.equal(tail[ends[b]], whole[last[b]]), b
    single, _ = run_attention(kn, None, lengths, [1] * 4, heads, kv_heads, head_dim, torch.float32, 71, window=window,
                              decode=True, force_generic=True, q_by_position=True)
    for b in range(len(lengths)):
        assert torch.equal(single[b], whole[last[b]]), b


def test_attention_reference_vectors(kn):
    """q = k = v = 0.1 over 256 keys gives 0.1, 0.05 over 1500 keys gives 0.05
    (internal/device/attention_test.go:10-94)."""
    for n, val, heads in ((256, 0.1, 8), (1500, 0.05, 1)):
        hd = 128
        blocks = (n + BS - 1) // BS
        kc = torch.full((blocks, heads, BS, hd), val, dtype=torch.float32, device=DEV)
        vc = torch.full((blocks, heads, hd, BS), val, dtype=torch.float32, device=DEV)
        table = torch.arange(blocks, dtype=torch.int32, device=DEV).view(1, -1)
        q = torch.full((1, heads * hd), val, dtype=torch.float32, device=DEV)
        out = torch.empty_like(q)
        kn.attention(q, out, heads, heads, hd, i32([n - 1]), i32([0]), i32([0]), i32([0, 1]), table, kc, vc, BS,
                     1 / math.sqrt(hd), 0, decode=True, max_len=n)
        assert float((out - val).abs().max()) < 1e-6


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rope_store_rotates_and_writes_the_right_rows(kn, dtype):
    heads, kv_heads, hd = 6, 3, 48
    freqs = plain.rope_frequencies(hd, 25000.0)
    pos = [0, 5, 63, 64, 200]
    rows = len(pos)
    width = (heads + 2 * kv_heads) * hd
    qkv = rnd((rows, width), 31, dtype)
    orig = qkv.clone()
    n_blocks = 6
    kc = torch.zeros((n_blocks, kv_heads, BS, hd), dtype=dtype, device=DEV)
    vc = torch.zeros((n_blocks, kv_heads, hd, BS), dtype=dtype, device=DEV)
    table = torch.tensor([[0, 0, 0, 0], [5, 2, 4, 1]], dtype=torch.int32, device=DEV)  # slot 1 is used
    q = qkv[:, : heads * hd]
    k = qkv[:, heads * hd : (heads + kv_heads) * hd]
    v = qkv[:, (heads + kv_heads) * hd :]
    kn.rope_store(q, k, v, heads, kv_heads, hd, freqs.to(DEV), i32(pos), i32([0] * rows), i32([1]), table, kc, vc, BS)
    tol = 2e-6 if dtype == torch.float32 else 5e-3
    want_q = plain.rope(orig[:, : heads * hd].cpu().view(rows, heads, hd), pos, freqs)
    assert rel_err(q.reshape(rows, heads, hd), want_q) < tol
    want_k = plain.rope(orig[:, heads * hd : (heads + kv_heads) * hd].cpu().view(rows, kv_heads, hd), pos, freqs)
    phys = [5, 2, 4, 1]
    written = torch.zeros_like(kc, dtype=torch.bool)
    for r, p in enumerate(pos):
        blk, off = phys[p // BS], p % BS
        assert rel_err(kc[blk, :, off, :], want_k[r]) < tol
        assert torch.equal(vc[blk, :, :, off], orig[r, (heads + kv_heads) * hd :].view(kv_heads, hd))
        written[blk, :, off, :] = True
    # writing position p changes row p only (internal/device/kvcache_test.go:88-104)
    assert float(kc[~written].abs().max()) == 0.0
    # the reference's own vector: hd 128, 32 heads, pos 5, theta 1e4, input i/100
    # (internal/device/rope_test.go:10-65)
    x = (torch.arange(32 * 128, dtype=torch.float32) / 100.0).view(1, -1).to(dtype).to(DEV)
    x0 = x.clone()
    f = plain.rope_frequencies(128, 10000.0)
    kn.rope_store(x, None, None, 32, 0, 128, f.to(DEV), i32([5]))
    assert float((x.double().cpu().view(1, 32, 128) - plain.rope(x0.cpu().view(1, 32, 128), [5], f)).abs().max()) \
        < (1e-4 if dtype == torch.float32 else 0.2)


@pytest.mark.parametrize("heads,kv_heads,hd", [(32, 8, 128), (6, 3, 48), (8, 2, 64)])
def test_rope_store_by_groups_of_eight_positions_writes_the_same_bits(kn, heads, kv_heads, hd):
    """The kernel for prompt rows (eight positions of a sequence a block, cos and sin from the step's table,
    V into the transposed cache in runs of eight positions) against the kernel that takes a row at a time:
    sequences that start at any position (a prompt's later portion), of any length, side by side in one step;
    q, the K cache and the V cache come out bit for bit the same, and nothing else in the caches is touched."""
    freqs = plain.rope_frequencies(hd, 500000.0).to(DEV)
    starts, lens = [0, 3, 64, 70, 5, 127, 8], [200, 1, 9, 130, 3, 2, 16]
    slots = [4, 2, 7, 1, 5, 3, 6]
    n_blocks, per_seq = 40, 4
    g = torch.Generator().manual_seed(9)
    table = torch.randperm(n_blocks, generator=g)[: 8 * per_seq].view(8, per_seq).to(torch.int32).to(DEV)
    pos, row_seq, cu = [], [], [0]
    for b, (st, n) in enumerate(zip(starts, lens)):
        pos += list(range(st, st + n))
        row_seq += [b] * n
        cu.append(cu[-1] + n)
    rows = len(pos)
    width = (heads + 2 * kv_heads) * hd
    qkv0 = rnd((rows, width), 33, torch.bfloat16)
    results = []
    for grouped in (False, True):
        qkv = qkv0.clone()
        kc = torch.full((n_blocks, kv_heads, BS, hd), 3.0, dtype=torch.bfloat16, device=DEV)
        vc = torch.full((n_blocks, kv_heads, hd, BS), 3.0, dtype=torch.bfloat16, device=DEV)
        q, k = qkv[:, : heads * hd], qkv[:, heads * hd : (heads + kv_heads) * hd]
        v = qkv[:, (heads + kv_heads) * hd :]
        extra = {}
        if grouped:
            cs = torch.empty((rows, hd // 2, 2), dtype=torch.float32, device=DEV)
            kn.rope_table(freqs, i32(pos), cs)
            extra = dict(cos_sin=cs, cu_rows=i32(cu))
        kn.rope_store(q, k, v, heads, kv_heads, hd, freqs, i32(pos), i32(row_seq), i32(slots), table, kc, vc, BS, **extra)
        results.append((qkv, kc, vc))
    for a, b in zip(*results):
        assert torch.equal(a, b)
    kc, vc = results[1][1], results[1][2]
    touched = torch.zeros((n_blocks, BS), dtype=torch.bool)
    for b, (st, n) in enumerate(zip(starts, lens)):
        for p in range(st, st + n):
            touched[int(table[slots[b], p // BS]), p % BS] = True
    assert bool((kc.cpu().permute(0, 2, 1, 3)[~touched] == 3.0).all())
    assert bool((vc.cpu().permute(0, 3, 1, 2)[~touched] == 3.0).all())


@pytest.mark.parametrize("heads,kv_heads,hd,pieces", [(32, 8, 128, 4), (6, 3, 48, 3), (8, 2, 64, 1), (3, 1, 16, 7)])
def test_rope_store_from_the_pieces_of_a_product_writes_the_same_bits(kn, heads, kv_heads, hd, pieces):
    """q, k and v as the float32 partial sums that a product leaves where it shares K over blocks: the kernel
    adds them in ascending order, rounds the sums to bfloat16 and rotates and stores as `rope_store` does with
    rows that were summed and rounded beforehand; q, the K cache and the V cache come out bit for bit the same."""
    freqs = plain.rope_frequencies(hd, 500000.0).to(DEV)
    starts, lens = [0, 3, 64, 70], [130, 1, 9, 60]
    slots = [4, 2, 7, 1]
    n_blocks, per_seq = 40, 4
    g = torch.Generator().manual_seed(10)
    table = torch.randperm(n_blocks, generator=g)[: 8 * per_seq].view(8, per_seq).to(torch.int32).to(DEV)
    pos, row_seq = [], []
    for b, (st, n) in enumerate(zip(starts, lens)):
        pos += list(range(st, st + n))
        row_seq += [b] * n
    rows = len(pos)
    width = (heads + 2 * kv_heads) * hd
    parts = rnd((pieces, rows, width), 34, torch.float32)
    total = parts[0].clone()
    for s in range(1, pieces):
        total = total + parts[s]
    qkv = total.bfloat16()
    caches = []
    for _ in range(2):
        caches.append((torch.full((n_blocks, kv_heads, BS, hd), 3.0, dtype=torch.bfloat16, device=DEV),
                       torch.full((n_blocks, kv_heads, hd, BS), 3.0, dtype=torch.bfloat16, device=DEV)))
    q, k = qkv[:, : heads * hd], qkv[:, heads * hd : (heads + kv_heads) * hd]
    v = qkv[:, (heads + kv_heads) * hd :]
    kn.rope_store(q, k, v, heads, kv_heads, hd, freqs, i32(pos), i32(row_seq), i32(slots), table, caches[0][0],
                  caches[0][1], BS)
    q_out = torch.empty((rows, heads * hd), dtype=torch.bfloat16, device=DEV)
    kn.rope_store_pieces(parts, q_out, heads, kv_heads, hd, freqs, i32(pos), i32(row_seq), i32(slots), table,
                         caches[1][0], caches[1][1], BS)
    assert torch.equal(q_out, q)
    assert torch.equal(caches[0][0], caches[1][0]) and torch.equal(caches[0][1], caches[1][1])


@pytest.mark.parametrize("head_dim,heads,kv_heads,lengths", [
    (128, 8, 2, [5000, 300, 40, 1025, 256, 257, 2, 3000]),            # one long sequence among short ones
    (64, 4, 1, [700, 64, 1, 1500, 1500, 513, 30, 31, 32, 33, 9000]),  # one kv head; 11 sequences
    (128, 4, 4, [600, 4700]),                                         # two sequences, no head shared
    (192, 6, 3, [2500, 10, 900]),                                     # (two waves a workgroup)
    (64, 8, 2, [260] * 3 + [3000] * 2 + [1] * 27),                    # 32 sequences, most of one token
    (128, 8, 2, [4000, 3500] + [300 + 7 * i for i in range(38)] + [1, 2, 64, 65] * 6),  # 64 sequences: four units each
    (64, 4, 4, [2500] + [90 + i for i in range(39)]),                 # 40 sequences
])
def test_decode_attention_that_shares_its_keys_out_by_the_true_lengths(kn, head_dim, heads, kv_heads, lengths):
    """With the hint that the lengths are uneven the workgroups of a decoding launch number the splits that hold
    keys through (whole splits first, then every sequence's last) and each takes one, whatever sequence it belongs
    to: against the plain implementation, against the launch without the hint (the same sums in another order),
    twice the same, the tickets back at zero; a far key that stands out is found in the long sequence.  Up to 64
    sequences (a lane of a wave looks after each), from 33 on with four units a sequence."""
    n = len(lengths)
    got, want = run_attention(kn, None, lengths, [1] * n, heads, kv_heads, head_dim, torch.bfloat16, 41, decode=True,
                              uneven=True)
    assert rel_err(got, want) < 8e-3
    for b in range(n):  # every sequence by itself: a short one is not hidden behind a long one's size
        assert rel_err(got[b], want[b]) < 1.2e-2, b
    plain_grid, _ = run_attention(kn, None, lengths, [1] * n, heads, kv_heads, head_dim, torch.bfloat16, 41, decode=True)
    assert rel_err(got, plain_grid.double().cpu()) < 8e-3
    again, _ = run_attention(kn, None, lengths, [1] * n, heads, kv_heads, head_dim, torch.bfloat16, 41, decode=True,
                             uneven=True)
    assert torch.equal(got, again)
    assert int(kn.tickets(torch.device('cuda', torch.cuda.current_device())).abs().max()) == 0
    longest = max(range(n), key=lambda b: lengths[b])
    got, want = run_attention(kn, None, lengths, [1] * n, heads, kv_heads, head_dim, torch.bfloat16, 43, decode=True,
                              uneven=True, standout=(longest, 77))
    assert rel_err(got, want) < 8e-3
    assert float(got[longest].float().mean()) > 6.0  # the values of key 77 (7.0) dominate the long sequence's row


@pytest.mark.parametrize("m", [1, 8, 16, 33, 64, 65, 300, 400])
@pytest.mark.parametrize("inner,k", [(16, 8), (328, 96), (1000, 264), (8200, 96), (14336, 4096), (1032, 512)])
def test_linear_with_fused_swiglu(kn, m, inner, k):
    """One kernel for silu(x Wg^T) * (x Wu^T), with gate and up rows interleaved in groups of 8
    (every kernel of the product has this epilogue: the GEMVs, the tiled and the pipelined ones)."""
    if inner == 14336 and m == 65:
        m = 130
    if inner == 1032 and m == 400:
        m, inner, k = 2048, 14336, 128  # 3.5 rounds of 256 x 256 tiles: the last half round goes as 128-column tiles
    x = rnd((m, k), 41, torch.bfloat16)
    gate, up = rnd((inner, k), 42, torch.bfloat16, 0.05), rnd((inner, k), 43, torch.bfloat16, 0.05)
    assert kn.linear_swiglu_supported(torch.bfloat16, 2 * inner, k)
    w = kn.interleave_gate_up(gate, up)
    out = torch.empty((m, inner), dtype=torch.bfloat16, device=DEV)
    kn.linear_swiglu(x, w, out)
    xd = x.double().cpu()
    want = plain.swiglu(xd @ gate.double().cpu().t(), xd @ up.double().cpu().t())
    assert rel_err(out, want) < 5e-3
    out32 = torch.empty((m, inner), dtype=torch.float32, device=DEV)
    kn.linear_swiglu(x, w, out32)
    assert rel_err(out32, want) < 2e-5


@pytest.mark.parametrize("heads,kv_heads,head_dim", [(32, 8, 128), (4, 2, 64), (16, 1, 64), (6, 3, 192)])
@pytest.mark.parametrize("window", [0, 100])
def test_decode_attention_with_rotation_and_cache_write_folded_in(kn, heads, kv_heads, head_dim, window):
    """One launch that rotates q and k, writes k and v into the cache and attends, against the two
    separate kernels (rope_store, then attention)."""
    dtype = torch.bfloat16
    lengths = [700, 64, 257, 1, 1300]
    assert kn.attention_folds_rope(dtype, heads, kv_heads, head_dim, BS)
    kc, vc, table, slots, dense = paged_cache(lengths, kv_heads, head_dim, dtype, 51)
    kc2, vc2 = kc.clone(), vc.clone()
    rows = len(lengths)
    width = (heads + 2 * kv_heads) * head_dim
    qkv = rnd((rows, width), 52, dtype)
    qkv2 = qkv.clone()
    pos = [n - 1 for n in lengths]
    freqs = plain.rope_frequencies(head_dim, 500000.0).to(DEV)
    cu = list(range(rows + 1))
    scale = 1.0 / math.sqrt(head_dim)
    need = kn.attention_workspace(dtype, rows, heads, kv_heads, head_dim, BS, True, max(lengths))
    ws = torch.empty(max(need, 1), dtype=torch.float32, device=DEV)

    def views(t):
        return t[:, : heads * head_dim], t[:, heads * head_dim : (heads + kv_heads) * head_dim], t[:, (heads + kv_heads) * head_dim :]

    q, k, v = views(qkv)
    out_a = torch.empty((rows, heads * head_dim), dtype=dtype, device=DEV)
    kn.rope_store(q, k, v, heads, kv_heads, head_dim, freqs, i32(pos), i32(range(rows)), i32(slots), table, kc, vc, BS)
    kn.attention(q, out_a, heads, kv_heads, head_dim, i32(pos), i32(range(rows)), i32(slots), i32(cu), table, kc, vc, BS,
                 scale, window, decode=True, max_len=max(lengths), workspace=ws)
    q2, k2, v2 = views(qkv2)
    cs = torch.empty((rows, head_dim // 2, 2), dtype=torch.float32, device=DEV)
    kn.rope_table(freqs, i32(pos), cs)
    ang = torch.tensor(pos, dtype=torch.float64)[:, None] * freqs.cpu()[None, :]
    assert float((cs[..., 0].cpu().double() - torch.cos(ang)).abs().max()) < 1e-6
    assert float((cs[..., 1].cpu().double() - torch.sin(ang)).abs().max()) < 1e-6
    out_b = torch.empty_like(out_a)
    kn.attention(q2, out_b, heads, kv_heads, head_dim, i32(pos), i32(range(rows)), i32(slots), i32(cu), table, kc2, vc2,
                 BS, scale, window, decode=True, max_len=max(lengths), workspace=ws, k_new=k2, v_new=v2, cos_sin=cs)
    assert torch.equal(kc, kc2) and torch.equal(vc, vc2)  # the same rows of the cache were written, with the same bits
    assert rel_err(out_b, out_a.double().cpu()) < 4e-3


@pytest.mark.parametrize("heads,kv_heads,head_dim,pieces", [(32, 8, 128, 4), (4, 2, 64, 2), (16, 1, 64, 7), (6, 3, 192, 3)])
@pytest.mark.parametrize("uneven", [False, True])
def test_decode_attention_that_adds_up_the_pieces_of_its_projections(kn, heads, kv_heads, head_dim, pieces, uneven):
    """The folded launch given q, k and v as float32 partial sums (what a product leaves that shares K over
    blocks) against the same launch given their sums rounded to bfloat16: the same bits, in the output and in
    the cache."""
    from longbow_quarrel_amd.kernels.hip import KernelLibraryError
    dtype = torch.bfloat16
    lengths = [700, 64, 257, 1, 1300, 2, 900]
    assert kn.attention_adds_pieces(dtype, heads, kv_heads, head_dim, BS)
    kc, vc, table, slots, dense = paged_cache(lengths, kv_heads, head_dim, dtype, 61)
    kc2, vc2 = kc.clone(), vc.clone()
    rows = len(lengths)
    width = (heads + 2 * kv_heads) * head_dim
    parts = rnd((pieces, rows, width), 62, torch.float32)
    whole = parts[0].clone()
    for i in range(1, pieces):  # in this order, as the launch adds them
        whole = whole + parts[i]
    whole = whole.to(dtype)
    pos = [n - 1 for n in lengths]
    freqs = plain.rope_frequencies(head_dim, 500000.0).to(DEV)
    cu = list(range(rows + 1))
    scale = 1.0 / math.sqrt(head_dim)
    need = kn.attention_workspace(dtype, rows, heads, kv_heads, head_dim, BS, True, max(lengths))
    ws = torch.empty(max(need, 1), dtype=torch.float32, device=DEV)
    cs = torch.empty((rows, head_dim // 2, 2), dtype=torch.float32, device=DEV)
    kn.rope_table(freqs, i32(pos), cs)

    def views(t):
        return t[:, : heads * head_dim], t[:, heads * head_dim : (heads + kv_heads) * head_dim], t[:, (heads + kv_heads) * head_dim :]

    outs = []
    for src, k_cache, v_cache, more in ((whole, kc, vc, {}),
                                        (parts[0], kc2, vc2, dict(pieces=pieces, piece_stride=parts.stride(0)))):
        q, k, v = views(src)
        out = torch.empty((rows, heads * head_dim), dtype=dtype, device=DEV)
        kn.attention(q, out, heads, kv_heads, head_dim, i32(pos), i32(range(rows)), i32(slots), i32(cu), table,
                     k_cache, v_cache, BS, scale, 0, decode=True, max_len=max(lengths), workspace=ws, k_new=k,
                     v_new=v, cos_sin=cs, uneven=uneven, **more)
        outs.append(out)
    assert torch.equal(kc, kc2) and torch.equal(vc, vc2)
    assert torch.equal(outs[0], outs[1])
    with pytest.raises(KernelLibraryError):  # pieces without the folded rotation: refused
        q, k, v = views(parts[0])
        kn.attention(q, outs[1], heads, kv_heads, head_dim, i32(pos), i32(range(rows)), i32(slots), i32(cu), table,
                     kc2, vc2, BS, scale, 0, decode=True, max_len=max(lengths), workspace=ws, pieces=pieces,
                     piece_stride=parts.stride(0))

