"""Each kernel alone against a plain PyTorch float32/float64 reference of the same
operation, at sizes other than the tiny models': widths and vocabularies that are no
powers of two, head sizes in steps of 16, any number of heads and groups, several page
sizes, windows.  Where random inputs would hide a fault the inputs are made so that it
shows: one far key whose score stands out, keys at a page's edge, a window's edge."""
import math

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from xyntetik_runner_amd.csrc.ops import load_ops
    return load_ops()


DEV = "cuda:0"
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def rel(got, want):
    return (got.double() - want.double()).abs().max().item() / max(want.double().abs().max().item(), 1e-30)


# ------------------------------------------------------------------ small kernels
@pytest.mark.parametrize("V,E", [(100, 72), (333, 4100), (77, 4104)])
@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
def test_embedding(ops, V, E, dt):
    table = torch.randn(V, E, device=DEV).to(DT[dt])
    ids = torch.tensor([0, V - 1, 5, -3, V, 17], dtype=torch.int32, device=DEV)
    got = ops.embedding(table, ids, scale=1.0)
    want = table.float()[torch.tensor([0, V - 1, 5, 0, 0, 17], device=DEV)]       # out of range reads row 0
    assert got.dtype == torch.float32 and torch.equal(got, want)
    assert torch.equal(ops.embedding(table, ids, scale=2.0), want * 2)
    if dt == "bfloat16":            # the same rows from the table in the matrix kernels' packed order
        packed = ops.pack_weight(table)
        assert (packed is not table) == (E % 8 == 0)            # (a width that is no multiple of 8 is not packed)
        assert torch.equal(ops.embedding(packed, ids, scale=1.0), want)


@pytest.mark.parametrize("n_words,blocks", [(4, 1), (1 << 20, 64), (12345 * 4, 2048), (3 * (1 << 20) + 4, 7)])
def test_stream_read_reads_every_word_once(ops, n_words, blocks):
    """The memory yardstick's kernel: the XOR it leaves is the XOR of all words of the buffer."""
    buf = torch.randint(-2 ** 31, 2 ** 31 - 1, (n_words,), dtype=torch.int32, device=DEV)
    got = ops.stream_read(buf, blocks).cpu().numpy().view(np.uint32)
    assert np.bitwise_xor.reduce(got) == np.bitwise_xor.reduce(buf.cpu().numpy().view(np.uint32))


@pytest.mark.parametrize("E", [8, 100, 4096, 5000])
@pytest.mark.parametrize("out", ["float32", "bfloat16"])
@pytest.mark.parametrize("wdt", ["float32", "bfloat16"])
def test_rmsnorm(ops, E, out, wdt):
    x = torch.randn(7, E, device=DEV) * 3
    w = (1 + 0.1 * torch.randn(E, device=DEV)).to(DT[wdt])
    for eps in (1e-5, 1e-2):
        want = x.double() / torch.sqrt((x.double() ** 2).mean(-1, keepdim=True) + eps) * w.double()
        got = ops.rmsnorm(x, w, eps, DT[out])
        assert rel(got, want) < (2e-6 if out == "float32" else 5e-3)
    rows = torch.tensor([6, 0, 3], dtype=torch.int32, device=DEV)
    got = ops.rmsnorm(x, w, 1e-5, DT[out], rows=rows)
    assert torch.equal(got, ops.rmsnorm(x, w, 1e-5, DT[out])[rows.long()])
    # eps placement shows on a near-zero row
    tiny = torch.full((1, E), 1e-4, device=DEV)
    got = ops.rmsnorm(tiny, None, 1e-6, torch.float32)
    assert abs(got[0, 0].item() - 1e-4 / math.sqrt(1e-8 + 1e-6)) < 1e-7


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
def test_silu_mul_add_convert_fill(ops, dt):
    T, F = 5, 301
    gu = (torch.randn(T, 2 * F, device=DEV) * 4).to(DT[dt])
    gu[0, 0] = -200.0
    g, u = gu[:, :F].double(), gu[:, F:].double()
    want = g / (1 + torch.exp(-g)) * u
    got = ops.silu_mul(gu)
    assert torch.isfinite(got.float()).all() and rel(got, want) < (1e-6 if dt == "float32" else 5e-3)
    x = torch.randn(T, F, device=DEV)
    y = torch.randn(T, F, device=DEV).to(DT[dt])
    want = x + y.float()
    ops.add_(x, y)
    assert torch.equal(x, want)
    c = ops.convert(x, torch.bfloat16)
    assert torch.equal(c, x.bfloat16()) and torch.equal(ops.convert(c, torch.float32), c.float())
    st = torch.randn(6, 3, 5, device=DEV)
    keep = st.clone()
    ops.fill_rows_(st, torch.tensor([4, 1], dtype=torch.int32, device=DEV), 2)
    assert (st[4] == 0).all() and (st[1] == 0).all() and torch.equal(st[[0, 2, 3, 5]], keep[[0, 2, 3, 5]])


# ------------------------------------------------------------------ matrix products
@pytest.mark.parametrize("M", [1, 5, 16, 17, 33, 64, 65, 130, 300])
@pytest.mark.parametrize("N,K", [(48, 64), (100, 72), (333, 264), (1000, 1032)])
def test_linear_bf16_mfma(ops, M, N, K):
    a = (torch.randn(M, K, device=DEV) * 0.5).bfloat16()
    w = (torch.randn(N, K, device=DEV) * 0.1).bfloat16()
    b = torch.randn(N, device=DEV) * 0.1
    want = a.double() @ w.double().T + b.double()
    assert rel(ops.linear(a, w, bias=b, out_dtype=torch.float32), want) < 1e-5       # 32-bit accumulation
    assert rel(ops.linear(a, w, bias=b), want) < 6e-3                                  # rounded once to bfloat16
    base = torch.randn(M, N, device=DEV)
    out = base.clone()
    ops.linear(a, w, out=out, accumulate=True)
    assert rel(out, base.double() + a.double() @ w.double().T) < 1e-5
    w2 = (torch.randn(2 * N, K, device=DEV) * 0.1).bfloat16()
    b2 = torch.randn(2 * N, device=DEV) * 0.1
    r = a.double() @ w2.double().T + b2.double()
    want = r[:, :N] / (1 + torch.exp(-r[:, :N])) * r[:, N:]
    assert rel(ops.linear_swiglu(a, w2, bias=b2), want) < 6e-3
    if M > 64:
        for variant in (12, 1014, 17, 26):               # tile shapes the dispatch may pick for other sizes
            assert rel(ops.linear(a, w, bias=b, out_dtype=torch.float32, variant=variant),
                       a.double() @ w.double().T + b.double()) < 1e-5


@pytest.mark.parametrize("variant", [51, 55, 58])
@pytest.mark.parametrize("M,N,K", [(65, 100, 256), (300, 333, 256), (513, 520, 1024), (256, 256, 4096), (300, 1352, 256)])
def test_four_wave_tile_kernels(ops, variant, M, N, K):
    """The 256x256, 256x128 and 128x128 tiles' kernels with four waves and a written order of instructions,
    by name (they refuse what they do not take): rows and columns that fill no tile, plain and packed
    weights, a bias, adding into the output, the gated epilogue; against the eight-wave kernel of
    the same tile the sums are the same to the bit (same products in the same order)."""
    from xyntetik_runner_amd.csrc.ops import KernelError
    eight_waves = {51: 114, 55: 112, 58: 117}[variant]            # (the same tile with the other loop)
    a = (torch.randn(M, K, device=DEV) * 0.5).bfloat16()
    w = (torch.randn(N, K, device=DEV) * 0.1).bfloat16()
    b = torch.randn(N, device=DEV) * 0.1
    want = a.double() @ w.double().T + b.double()
    for wt in (w, ops.pack_weight(w)):
        got = ops.linear(a, wt, bias=b, out_dtype=torch.float32, variant=variant)
        assert rel(got, want) < 1e-5
        assert torch.equal(got, ops.linear(a, wt, bias=b, out_dtype=torch.float32, variant=eight_waves))
        # the same tiles in the other orders of workgroups (side by side along the rows; by XCD, with
        # column tiles that are no multiple of 8: workgroups without a tile leave)
        for order in (1000, 2000):
            assert torch.equal(got, ops.linear(a, wt, bias=b, out_dtype=torch.float32, variant=order + variant))
        assert rel(ops.linear(a, wt, bias=b, variant=variant), want) < 6e-3
    base = torch.randn(M, N, device=DEV)
    out = base.clone()
    ops.linear(a, w, out=out, accumulate=True, variant=variant)
    assert rel(out, base.double() + a.double() @ w.double().T) < 1e-5
    w2 = (torch.randn(2 * N, K, device=DEV) * 0.1).bfloat16()
    b2 = torch.randn(2 * N, device=DEV) * 0.1
    r = a.double() @ w2.double().T + b2.double()
    want = r[:, :N] / (1 + torch.exp(-r[:, :N])) * r[:, N:]
    for wt in (w2, ops.pack_weight(w2, gated=True)):
        assert rel(ops.linear_swiglu(a, wt, bias=b2, variant=variant), want) < 6e-3
    # what they do not take is refused by name, and taken by the eight-wave kernel when the tile is asked for
    a2 = (torch.randn(M, 72, device=DEV) * 0.5).bfloat16()
    w3 = (torch.randn(N, 72, device=DEV) * 0.1).bfloat16()
    with pytest.raises(KernelError, match="four-wave"):
        ops.linear(a2, w3, variant=variant)
    assert rel(ops.linear(a2, w3, out_dtype=torch.float32, variant={51: 14, 55: 12, 58: 17}[variant]), a2.double() @ w3.double().T) < 1e-5


@pytest.mark.parametrize("M", [8, 40, 300])
def test_gated_product_with_gates_far_from_zero(ops, M):
    """Gate values of -200 and +200 through the fused epilogues: the weight-streaming kernel's
    (8 rows), the kernel's that adds up K ranges (40 rows) and the tile kernel's, which uses the
    hardware's 2^x and reciprocal (300 rows).  act(-200) * up is 0 and no NaN
    (src/model.c:4442-4452), act(200) is 200."""
    from xyntetik_runner_amd.csrc.ops import PackedWeight
    K, F = 64, 96
    a = torch.ones(M, K, device=DEV).bfloat16()
    wg = torch.empty(F, K, device=DEV)
    wg[:F // 2] = -200.0 / K
    wg[F // 2:] = 200.0 / K
    w2 = torch.cat([wg, torch.randn(F, K, device=DEV) * 0.1]).bfloat16()
    up = a.double() @ w2[F:].double().T
    for w in (w2, ops.pack_weight(w2, gated=True)):
        got = ops.linear_gated(a, w, activation="silu").float()
        assert torch.isfinite(got).all()
        assert (got[:, :F // 2] == 0).all()
        assert rel(got[:, F // 2:], 200.0 * up[:, F // 2:]) < 6e-3
    assert isinstance(ops.pack_weight(w2, gated=True), PackedWeight)
    with pytest.raises(Exception, match="not built into the kernels"):
        ops.linear_gated(a, w2, activation="no-such-activation")


@pytest.mark.parametrize("M", [8, 40, 300])
@pytest.mark.parametrize("first,width", [(0, 128), (4, 136), (3, 131), (2, 130)])
def test_linear_into_columns_of_a_wider_matrix(ops, M, first, width):
    """The output is a run of columns of a wider matrix: rows that begin 16 bytes aligned or not,
    row strides that are multiples of 4 or not (the tile kernel writes 4 columns a lane only
    where it may); what lies beside the run stays as it was."""
    N, K = 96, 80
    a = (torch.randn(M, K, device=DEV) * 0.5).bfloat16()
    w = (torch.randn(N, K, device=DEV) * 0.1).bfloat16()
    want = a.double() @ w.double().T
    for dt, tol in ((torch.float32, 1e-5), (torch.bfloat16, 6e-3)):
        big = torch.full((M, width), 7.0, device=DEV, dtype=dt)
        ops.linear(a, w, out=big[:, first:first + N])
        assert rel(big[:, first:first + N], want) < tol
        assert (big[:, :first] == 7).all() and (big[:, first + N:] == 7).all()
    big = torch.randn(M, width, device=DEV)
    keep = big.clone()
    ops.linear(a, w, out=big[:, first:first + N], accumulate=True)
    assert rel(big[:, first:first + N], keep[:, first:first + N].double() + want) < 1e-5
    assert torch.equal(big[:, :first], keep[:, :first]) and torch.equal(big[:, first + N:], keep[:, first + N:])


@pytest.mark.parametrize("M", [1, 8, 16, 17, 64, 65, 300])
@pytest.mark.parametrize("N,K", [(48, 64), (100, 72), (333, 264), (1000, 1032), (16, 8)])
def test_linear_packed_weights_give_the_same(ops, M, N, K):
    """Weights in the kernels' own order (1 KB blocks, zero padding) against the same weights
    row-major: the same sums in the same order, so the same bits; and against float64."""
    from xyntetik_runner_amd.csrc.ops import PackedWeight
    a = (torch.randn(M, K, device=DEV) * 0.5).bfloat16()
    w = (torch.randn(N, K, device=DEV) * 0.1).bfloat16()
    b = torch.randn(N, device=DEV) * 0.1
    pw = ops.pack_weight(w)
    assert isinstance(pw, PackedWeight) and pw.shape == (N, K)
    blocks = pw.data.cpu()
    n, k = 16 * (N // 16) + min(N % 16, 3) - (1 if N % 16 == 0 else 0), 8 * (K // 8 - 1)   # some row and chunk that exist
    assert torch.equal(blocks[n // 16, k // 32, n % 16, k % 32:k % 32 + 8], w[n, k:k + 8].cpu())
    if N % 16:
        assert (blocks[-1, :, N % 16:, :] == 0).all()                   # rows that do not exist
    if K % 32:
        assert (blocks[:, -1, :, K % 32:] == 0).all()                   # nor columns
    want = a.double() @ w.double().T + b.double()
    got = ops.linear(a, pw, bias=b, out_dtype=torch.float32)
    assert rel(got, want) < 1e-5
    assert torch.equal(got, ops.linear(a, w, bias=b, out_dtype=torch.float32))
    base = torch.randn(M, N, device=DEV)
    o1, o2 = base.clone(), base.clone()
    ops.linear(a, pw, out=o1, accumulate=True)
    ops.linear(a, w, out=o2, accumulate=True)
    assert torch.equal(o1, o2) and rel(o1, base.double() + a.double() @ w.double().T) < 1e-5
    F = 16 * max(1, N // 16)                                            # gate and up rows: heights in steps of 16
    w2 = (torch.randn(2 * F, K, device=DEV) * 0.1).bfloat16()
    b2 = torch.randn(2 * F, device=DEV) * 0.1
    pw2 = ops.pack_weight(w2, gated=True)
    assert isinstance(pw2, PackedWeight)
    r = a.double() @ w2.double().T + b2.double()
    got = ops.linear_swiglu(a, pw2, bias=b2)
    assert rel(got, r[:, :F] / (1 + torch.exp(-r[:, :F])) * r[:, F:]) < 6e-3
    assert torch.equal(got, ops.linear_swiglu(a, w2, bias=b2))


@pytest.mark.parametrize("M", [1, 5, 16])
@pytest.mark.parametrize("E,F,K", [(64, 96, 48), (200, 112, 72), (4096, 1024, 264), (72, 70000, 40), (5120, 8200, 256)])
@pytest.mark.parametrize("wdtype", [torch.float32, torch.bfloat16])
def test_rmsnorm_folded_into_the_products_around_it(ops, M, E, F, K, wdtype):
    """residual += a @ w^T; h = rmsnorm(residual); y = h @ w2^T.  With the norm folded in, the
    first product writes the weighted rows and partial sums of squares and the second applies
    the scale: the residual keeps the same bits, y agrees with the norm done in 64-bit, and
    neither depends on other rows of the batch."""
    from xyntetik_runner_amd.csrc.ops import UnscaledRows
    torch.manual_seed(M * 1000 + E)
    a = (torch.randn(M, K, device=DEV) * 0.5).bfloat16()
    w = ops.pack_weight((torch.randn(E, K, device=DEV) * 0.1).bfloat16())
    nw = (1 + 0.2 * torch.randn(E, device=DEV)).to(wdtype)
    w2 = (torch.randn(F, E, device=DEV) * 0.05).bfloat16()
    bias2 = torch.randn(F, device=DEV) * 0.1
    res0 = torch.randn(M, E, device=DEV) * torch.linspace(0.1, 30, M, device=DEV)[:, None]   # rows of very different size
    eps = 1e-5

    r_sep = res0.clone()
    h_sep = ops.linear_add_rmsnorm(a, w, r_sep, nw, eps, torch.bfloat16)
    assert isinstance(h_sep, torch.Tensor)
    r_fold = res0.clone()
    h = ops.linear_add_rmsnorm(a, w, r_fold, nw, eps, torch.bfloat16, defer=True)
    assert isinstance(h, UnscaledRows) and h.shape == (M, E)
    assert torch.equal(r_fold, r_sep)
    x = r_fold.double()
    assert rel(h.sumsq[:, :M].sum(0), (x * x).sum(1)) < 1e-5
    want_h = x * torch.rsqrt((x * x).mean(1, keepdim=True) + eps) * nw.double()
    y = ops.linear(h, w2, bias=bias2, out_dtype=torch.float32)
    y_sep = ops.linear(h_sep, w2, bias=bias2, out_dtype=torch.float32)
    want = want_h @ w2.double().T + bias2.double()
    # (either way the normed rows are rounded to bfloat16 once, so the errors are alike)
    assert rel(y, want) < 6e-3 and rel(y_sep, want) < 6e-3
    pw2 = ops.pack_weight(w2)
    assert torch.equal(ops.linear(h, pw2, bias=bias2, out_dtype=torch.float32), y)
    if F % 32 == 0:
        g = want_h @ w2.double().T
        got = ops.linear_swiglu(h, ops.pack_weight(w2, gated=True))
        assert rel(got, g[:, :F // 2] / (1 + torch.exp(-g[:, :F // 2])) * g[:, F // 2:]) < 8e-3
    # a chain: the second product adds into the residual and hands on to a third
    w3 = (torch.randn(E, F, device=DEV) * 0.05).bfloat16()
    h2 = ops.linear_add_rmsnorm(ops.linear(h, w2), w3, r_fold, nw, eps, torch.bfloat16, defer=True)
    r2 = r_sep.clone()
    ops.linear(ops.linear(h_sep, w2), w3, out=r2, accumulate=True)
    want_r2 = x + (want_h @ w2.double().T) @ w3.double().T
    assert isinstance(h2, UnscaledRows) and rel(r_fold, want_r2) < 1e-2
    assert rel(r2, want_r2) < 1e-2
    # a row's result does not depend on the rows beside it
    if M > 1:
        r1 = res0[M - 1:].clone()
        h1 = ops.linear_add_rmsnorm(a[M - 1:], w, r1, nw, eps, torch.bfloat16, defer=True)
        assert torch.equal(r1, r_sep[M - 1:]) and torch.equal(h1.data, h.data[M - 1:])
        assert torch.equal(ops.linear(h1, w2, bias=bias2, out_dtype=torch.float32), y[M - 1:])
    # where the folded form is not served, the same call runs the norm's own kernel
    a17 = (torch.randn(17, K, device=DEV) * 0.5).bfloat16()
    assert isinstance(ops.linear_add_rmsnorm(a17, w, torch.zeros(17, E, device=DEV), nw, eps, torch.bfloat16, defer=True),
                      torch.Tensor)
    with pytest.raises(Exception, match="at most 16|MFMA"):
        ops.linear(UnscaledRows(torch.zeros(17, E, device=DEV).bfloat16(), h.sumsq, eps), w2)


def test_linear_whose_tiles_do_not_fill_the_last_round(ops):
    """314 tiles of 256x256 make a full round of 256 and a round of 58: the columns of the full
    round go to that tile and the rest to a second launch with a smaller tile.  Every column
    must be computed once (an accumulating epilogue would show a second time), also where the
    two launches meet and at the ragged end."""
    torch.manual_seed(5)
    M, N, K = 512, 40008, 64
    a = (torch.randn(M, K, device=DEV) * 0.5).bfloat16()
    w = (torch.randn(N, K, device=DEV) * 0.1).bfloat16()
    b = torch.randn(N, device=DEV) * 0.1
    want = a.double() @ w.double().T
    for wt in (w, ops.pack_weight(w)):
        assert rel(ops.linear(a, wt, bias=b, out_dtype=torch.float32), want + b.double()) < 1e-5
        base = torch.randn(M, N, device=DEV)
        out = base.clone()
        ops.linear(a, wt, out=out, accumulate=True)
        assert rel(out, base.double() + want) < 1e-5
        assert rel(out[:, 32768 - 300:32768 + 300], (base.double() + want)[:, 32768 - 300:32768 + 300]) < 1e-5
    F = 20000
    w2 = (torch.randn(2 * F, K, device=DEV) * 0.1).bfloat16()
    r = a.double() @ w2.double().T
    got = ops.linear_swiglu(a, ops.pack_weight(w2, gated=True))
    assert rel(got, r[:, :F] / (1 + torch.exp(-r[:, :F])) * r[:, F:]) < 6e-3


@pytest.mark.parametrize("M", [17, 33, 64, 100, 300])
@pytest.mark.parametrize("E,K", [(64, 48), (200, 520), (4096, 1024), (5120, 264)])
@pytest.mark.parametrize("wdtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("bias", [False, True])
def test_rmsnorm_by_the_kernel_that_adds_up_a_split_product(ops, M, E, K, wdtype, bias):
    """17 to 64 rows, and more where the product's tiles are few enough for K to be split:
    residual += a @ w^T (+ bias) and the norm of the result from the product and
    one more kernel; against the product and the norm's own kernel (the residual to the bit when
    the K ranges are the same, else to rounding) and against float64."""
    torch.manual_seed(M + E)
    a = (torch.randn(M, K, device=DEV) * 0.5).bfloat16()
    w = ops.pack_weight((torch.randn(E, K, device=DEV) * 0.1).bfloat16())
    b = torch.randn(E, device=DEV) * 0.2 if bias else None
    nw = (1 + 0.2 * torch.randn(E, device=DEV)).to(wdtype)
    res0 = torch.randn(M, E + 4, device=DEV)[:, :E] * torch.linspace(0.1, 30, M, device=DEV)[:, None]
    eps = 1e-6
    r1, r2 = res0.clone(), res0.clone()
    assert r1.stride(0) == E
    h1 = ops.linear_add_rmsnorm(a, w, r1, nw, eps, torch.bfloat16, bias=b)
    ops.fold_norms = False
    try:
        h2 = ops.linear_add_rmsnorm(a, w, r2, nw, eps, torch.bfloat16, bias=b)
    finally:
        ops.fold_norms = True
    assert isinstance(h1, torch.Tensor) and h1.dtype == torch.bfloat16 and h1.shape == (M, E)
    from xyntetik_runner_amd.csrc.ops import PackedWeight
    wd = w.data if isinstance(w, PackedWeight) else w
    x = res0.double() + a.double() @ _unpack(wd, E, K).double().T + (b.double() if bias else 0)
    assert rel(r1, x) < 1e-5 and rel(r2, x) < 1e-5
    want = x * torch.rsqrt((x * x).mean(1, keepdim=True) + eps) * nw.double()
    assert rel(h1, want) < 6e-3 and rel(h2, want) < 6e-3
    assert rel(h1, h2.float()) < 8e-3           # a bfloat16 rounding apart at most


def _unpack(data, N, K):
    """A packed weight back in rows."""
    if data.dim() == 2:
        return data
    return data.permute(0, 2, 1, 3).reshape(data.shape[0] * 16, data.shape[1] * 32)[:N, :K]


def test_long_products_with_few_tiles_are_split_over_k(ops):
    """1024 x 4096 x 14336 (a down product): 128 tiles of 256x128 (or 64 of 256x256) would fill half
    the chip or less, so K is split and a second kernel adds the ranges into the residual stream;
    asked for the norm that follows, that kernel writes it too and the norm's own kernel is not
    launched."""
    torch.manual_seed(11)
    M, N, K = 1024, 4096, 14336
    a = (torch.randn(M, K, device=DEV) * 0.3).bfloat16()
    w = (torch.randn(N, K, device=DEV) * 0.05).bfloat16()
    pw = ops.pack_weight(w)
    b = torch.randn(N, device=DEV) * 0.1
    nw = (1 + 0.2 * torch.randn(N, device=DEV)).bfloat16()
    base = torch.randn(M, N, device=DEV)
    x = base.double() + a.double() @ w.double().T + b.double()
    out = base.clone()
    ops.linear(a, pw, bias=b, out=out, accumulate=True)
    assert rel(out, x) < 1e-5
    launches = [0]
    plain_norm = ops.rmsnorm
    def counting(*args, **kw):
        launches[0] += 1
        return plain_norm(*args, **kw)
    out2 = base.clone()
    try:
        ops.rmsnorm = counting
        h = ops.linear_add_rmsnorm(a, pw, out2, nw, 1e-5, torch.bfloat16, bias=b)
    finally:
        del ops.rmsnorm
    assert launches[0] == 0 and rel(out2, x) < 1e-5      # (the product alone may take other tiles: another order of 32-bit sums)
    want = x * torch.rsqrt((x * x).mean(1, keepdim=True) + 1e-5) * nw.double()
    assert h.dtype == torch.bfloat16 and rel(h, want) < 6e-3
    # a product the library does not split: the same call runs the norm's kernel
    a2 = (torch.randn(300, 64, device=DEV)).bfloat16()
    w2 = (torch.randn(N, 64, device=DEV) * 0.1).bfloat16()
    r2 = torch.randn(300, N, device=DEV)
    x2 = r2.double() + a2.double() @ w2.double().T
    try:
        ops.rmsnorm = counting
        h2 = ops.linear_add_rmsnorm(a2, w2, r2, nw, 1e-5, torch.bfloat16)
    finally:
        del ops.rmsnorm
    assert launches[0] == 1 and rel(r2, x2) < 1e-5
    assert rel(h2, x2 * torch.rsqrt((x2 * x2).mean(1, keepdim=True) + 1e-5) * nw.double()) < 6e-3


def test_pack_weight_leaves_what_the_mfma_kernels_do_not_take(ops):
    w = torch.randn(40, 20, device=DEV).bfloat16()                      # width no multiple of 8
    assert ops.pack_weight(w) is w
    w = torch.randn(40, 24, device=DEV)                                 # 32-bit
    assert ops.pack_weight(w) is w
    w = torch.randn(2 * 24, 16, device=DEV).bfloat16()                  # gate and up rows of 24: not in steps of 16
    assert ops.pack_weight(w, gated=True) is w and not isinstance(ops.pack_weight(w), torch.Tensor)
    from xyntetik_runner_amd.csrc.ops import KernelError
    with pytest.raises(KernelError):                                    # a packed weight has no 32-bit kernel to fall back to
        ops.linear(torch.randn(3, 16, device=DEV), ops.pack_weight(w))


@pytest.mark.parametrize("M,N,K", [(1, 7, 5), (9, 100, 77), (70, 65, 130)])
@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
def test_linear_plain_kernel(ops, M, N, K, dt):
    """Sizes the MFMA kernels refuse (K not a multiple of 8) and the whole 32-bit path."""
    a = torch.randn(M, K, device=DEV).to(DT[dt])
    w = torch.randn(N, K, device=DEV).to(DT[dt])
    b = torch.randn(N, device=DEV)
    want = a.double() @ w.double().T + b.double()
    assert rel(ops.linear(a, w, bias=b, out_dtype=torch.float32), want) < 2e-6
    base = torch.randn(M, N, device=DEV)
    out = base.clone()
    ops.linear(a, w, out=out, accumulate=True)
    assert rel(out, base.double() + a.double() @ w.double().T) < 2e-6


@pytest.mark.parametrize("M,N,K", [(1, 7, 8), (3, 50, 260), (8, 1000, 4096), (16, 33, 14336), (13, 65, 1028), (2, 128256 // 16, 64)])
def test_linear_32bit_few_rows(ops, M, N, K):
    """Up to 16 rows of 32-bit operands take the kernel that streams the weights (a wave 8 weight rows):
    against the float64 product, with bias, accumulation, a bfloat16 result and rows that are a view
    of a wider matrix; and a row's result is bit for bit the same whatever rows are beside it."""
    torch.manual_seed(M * 1000 + N)
    wide = torch.randn(M, K + 8, device=DEV)
    a = wide[:, :K]                                   # row stride K + 8
    w = torch.randn(N, K, device=DEV)
    b = torch.randn(N, device=DEV)
    want = a.double() @ w.double().T + b.double()
    got = ops.linear(a, w, bias=b, out_dtype=torch.float32)
    assert rel(got, want) < 2e-6
    base = torch.randn(M, N, device=DEV)
    out = base.clone()
    ops.linear(a, w, out=out, accumulate=True)
    assert rel(out, base.double() + a.double() @ w.double().T) < 2e-6
    assert rel(ops.linear(a, w, bias=b, out_dtype=torch.bfloat16).float(), want) < 6e-3
    alone = ops.linear(a[:1].contiguous(), w, bias=b, out_dtype=torch.float32)
    assert torch.equal(alone[0], got[0])
    if M < 16:                                        # and whatever kernel instance (1, 4, 8 or 16 rows) serves it
        more = torch.cat([a, torch.randn(16 - M, K, device=DEV)]).contiguous()
        assert torch.equal(ops.linear(more, w, bias=b, out_dtype=torch.float32)[:M], got)


def test_linear_32bit_sum_order_changes_at_17_rows_and_both_are_close(ops):
    """Up to 16 rows are summed by the streaming kernel, 17 and more by the tile kernel, in another
    order: over the 14,336 columns of the widest product both stay within 1e-6 of the float64
    product, and so does their difference for the same row."""
    torch.manual_seed(5)
    K, N = 14336, 96
    a = torch.randn(17, K, device=DEV)
    w = torch.randn(N, K, device=DEV) * 0.02
    want = a.double() @ w.double().T
    few = ops.linear(a[:16].contiguous(), w, out_dtype=torch.float32)
    many = ops.linear(a, w, out_dtype=torch.float32)
    assert rel(few, want[:16]) < 1e-6 and rel(many, want) < 1e-6
    assert rel(few, many[:16]) < 1e-6
    assert not torch.equal(few, many[:16])          # (if this ever holds, the header's caveat can go)


def test_linear_one_hot_rows_pick_weight_rows(ops):
    """A one-hot input returns the matching weight column: a transposed or mis-strided operand fails."""
    N, K = 96, 64
    w = torch.randn(N, K, device=DEV).bfloat16()
    for M in (3, 100):
        a = torch.zeros(M, K, device=DEV).bfloat16()
        cols = [(7 * i + 3) % K for i in range(M)]
        for i, c in enumerate(cols):
            a[i, c] = 1.0
        got = ops.linear(a, w, out_dtype=torch.float32)
        assert torch.equal(got, w.float()[:, cols].T.contiguous())


def test_linear_refuses_bad_operands(ops):
    from xyntetik_runner_amd.csrc.ops import KernelError
    a = torch.randn(4, 16, device=DEV).bfloat16()
    with pytest.raises(KernelError):
        ops.linear(a, torch.randn(8, 24, device=DEV).bfloat16())
    with pytest.raises(KernelError):
        ops.linear(a, torch.randn(8, 16, device=DEV))
    with pytest.raises(KernelError):
        ops.linear(a.cpu(), torch.randn(8, 16).bfloat16())


# ------------------------------------------------------------------ rotary + cache write + attention
class FakeCtx:
    """The part of a step's context that the attention kernels read."""

    def __init__(self, starts, q_lens, tables, page_size, cta_tiles=None):
        from xyntetik_runner_amd.engine.batch import plan_attention, AttentionPlan
        self.starts, self.q_lens = list(starts), list(q_lens)
        self.cta_tiles = cta_tiles
        pos, rot, cu = [], [], [0]
        for b, (s, n) in enumerate(zip(starts, q_lens)):
            pos += list(range(s, s + n)); rot += [b] * n; cu.append(cu[-1] + n)
        i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
        self.positions, self.req_of_token, self.cu_q, self.starts_dev = i32(pos), i32(rot), i32(cu), i32(list(starts))
        width = max(len(t) for t in tables)
        tab = torch.full((len(tables), width), -1, dtype=torch.int32)
        for b, t in enumerate(tables):
            tab[b, :len(t)] = torch.tensor(t, dtype=torch.int32)
        self._table = tab.to(DEV)
        self._plan_fn, self._Plan = plan_attention, AttentionPlan

    def block_table(self, group):
        return self._table

    def attention_plan(self, group, G, window, Hk, page_size=64):
        cta, items, jobs, n_slots = self._plan_fn(self.starts, self.q_lens, G, window, Hk, page_size,
                                                  cta_tiles=self.cta_tiles)
        it = torch.tensor([v for i in cta + items for v in i], dtype=torch.int32, device=DEV)
        jb = torch.tensor([v for j in jobs for v in j], dtype=torch.int32, device=DEV) if jobs else None
        return self._Plan(it, len(items), jb, len(jobs), n_slots, len(cta))


def scatter_pages(n_req_lens, page_size, seed):
    """Random, interleaved pages for each request (never page 0)."""
    rng = np.random.default_rng(seed)
    need = [-(-n // page_size) for n in n_req_lens]
    perm = rng.permutation(sum(need) + 3) + 1
    tables, k = [], 0
    for n in need:
        tables.append([int(p) for p in perm[k:k + n]]); k += n
    return tables, int(perm.max()) + 1


def ref_rope(x, pos, inv_freq, interleaved):
    T, H, D = x.shape
    half = inv_freq.numel()
    # the angle is a 32-bit product, as the kernel's and the reference's is (position x frequency
    # in float); its cosine and sine, and the rotation, in float64
    ang = (pos.float()[:, None] * inv_freq.float()[None, :]).double()
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    y = x.double().clone()
    i0 = torch.arange(half) * 2 if interleaved else torch.arange(half)
    i1 = i0 + 1 if interleaved else i0 + half
    y[..., i0] = x.double()[..., i0] * c - x.double()[..., i1] * s
    y[..., i1] = x.double()[..., i0] * s + x.double()[..., i1] * c
    return y


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,Hk,D,rot,inter", [(4, 2, 16, 16, False), (3, 1, 48, 32, False), (6, 3, 80, 80, True), (8, 8, 128, 64, True)])
@pytest.mark.parametrize("ps,starts,q_lens", [(8, [0, 13, 40], [9, 3, 1]), (64, [5, 64, 200, 0], [40, 17, 1, 8]),
                                              (4, [2, 9], [7, 6])])
def test_rope_kv_write(ops, dt, H, Hk, D, rot, inter, ps, starts, q_lens):
    """Portions that bring whole aligned groups of 8 positions (their values go to the transposed
    cache 8 at a time), groups cut at either end, single tokens, pages smaller than a group."""
    tables, n_pages = scatter_pages([s + n for s, n in zip(starts, q_lens)], ps, 1)
    ctx = FakeCtx(starts, q_lens, tables, ps)
    T = sum(q_lens)
    Q, K = H * D, Hk * D
    qkv = torch.randn(T, Q + 2 * K + 5, device=DEV)[:, :Q + 2 * K]          # a row stride that is not the width
    inv = (10000.0 ** (-torch.arange(rot // 2, dtype=torch.float64) * 2 / rot)).float().to(DEV)
    q_out = torch.empty(T, Q, device=DEV, dtype=DT[dt])
    kc = torch.full((n_pages, Hk, ps, D), float("nan"), device=DEV, dtype=DT[dt])
    vc = torch.full((n_pages, Hk, D, ps), float("nan"), device=DEV, dtype=DT[dt])
    ops.rope_kv_write(qkv[:, :Q], qkv[:, Q:Q + K], qkv[:, Q + K:], q_out, kc, vc, ctx.positions, ctx.req_of_token,
                      ctx.block_table(0), inv, H, Hk, D, rot, inter, 1.0, ps)
    pos = ctx.positions.cpu()
    want_q = ref_rope(qkv[:, :Q].cpu().reshape(T, H, D), pos, inv.cpu(), inter)
    want_k = ref_rope(qkv[:, Q:Q + K].cpu().reshape(T, Hk, D), pos, inv.cpu(), inter)
    tol = 2e-6 if dt == "float32" else 5e-3
    assert rel(q_out.cpu().reshape(T, H, D), want_q) < tol
    written = torch.zeros(n_pages, ps, dtype=torch.bool)
    t = 0
    for b, (s, n) in enumerate(zip(starts, q_lens)):
        for p in range(s, s + n):
            page, off = tables[b][p // ps], p % ps
            assert rel(kc[page, :, off, :].cpu(), want_k[t]) < tol
            assert rel(vc[page, :, :, off].cpu(), qkv[t, Q + K:].cpu().reshape(Hk, D).to(DT[dt])) == 0   # values as they are
            written[page, off] = True
            t += 1
    assert torch.isnan(kc.float().cpu().permute(0, 2, 1, 3)[~written]).all()      # nothing else was touched
    assert torch.isnan(vc.float().cpu().permute(0, 3, 1, 2)[~written]).all()
    if rot < D:                                                               # channels beyond the rotary width pass through
        assert torch.equal(q_out.cpu().reshape(T, H, D)[..., rot:], qkv[:, :Q].cpu().reshape(T, H, D)[..., rot:].to(DT[dt]))


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,Hk,D,rot,inter", [(4, 2, 16, 16, False), (3, 1, 48, 32, False), (6, 3, 80, 80, True),
                                               (8, 8, 128, 64, True), (5, 1, 128, 128, False), (2, 2, 32, 0, False)])
@pytest.mark.parametrize("ps,starts,q_lens", [(16, [0, 13, 40], [9, 3, 1]), (64, [70], [1]), (8, [2, 9, 100, 7], [5, 6, 1, 4]),
                                              (16, [3, 0], [30, 8]), (16, [5, 0, 77], [60, 20, 3]),
                                              (16, [3, 0, 8, 21], [290, 200, 70, 1]), (64, [64], [520]),
                                              (32, [3, 0, 8], [200, 70, 30]), (64, [1000], [511])])
@pytest.mark.parametrize("bias", [False, True])
def test_projection_with_rotation_and_cache_write(ops, dt, H, Hk, D, rot, inter, ps, starts, q_lens, bias):
    check_projection_with_rotation_and_cache_write(ops, dt, H, Hk, D, rot, inter, ps, starts, q_lens, bias, 72)


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("q_lens", [[100, 30], [20, 9], [300], [70, 200, 115]])
def test_projection_with_rotation_and_cache_write_of_a_product_split_over_k(ops, dt, q_lens):
    """The same with a width of 1,024, where the products of 17 to 511 rows are split over K
    (8 to 32 tiles of 128 columns for 256 compute units) and the kernel that adds the ranges up
    rotates and caches."""
    starts = [5, 0, 64][:len(q_lens)]
    check_projection_with_rotation_and_cache_write(ops, dt, 4, 2, 64, 64, False, 64, starts, q_lens, True, 1024)


@pytest.mark.parametrize("variant", [51, 55, 114, 112])
@pytest.mark.parametrize("H,Hk,D,rot,inter", [(4, 2, 64, 64, False), (3, 1, 48, 32, False), (2, 1, 80, 80, True), (5, 1, 128, 128, False)])
def test_projection_with_rotation_in_the_tile_kernels_by_name(ops, variant, H, Hk, D, rot, inter):
    """From 512 rows the tile kernel rotates and caches its own result: the four-wave kernels of the
    256x256 and 256x128 tiles (16 and 8 tiles of 32x32 a wave) and the eight-wave ones, by name, with
    heads that straddle the waves' tiles."""
    check_projection_with_rotation_and_cache_write(ops, "bfloat16", H, Hk, D, rot, inter, 16, [5, 0], [530, 70], True, 256, variant=variant)


def check_projection_with_rotation_and_cache_write(ops, dt, H, Hk, D, rot, inter, ps, starts, q_lens, bias, E, variant=0):
    """q, k and v from one product, rotated and cached.  Up to 16 bfloat16 rows the product's own
    kernel does all of it (with the weight's rows in paired order where a pair is (j, j + rot/2)),
    up to 511 the kernel that adds the product's K ranges up, from 512 the tile kernel;
    32-bit runs the product and the rotation kernel.  Both against float64 from
    the weights in their natural order; and the two bfloat16 ways against each other."""
    from xyntetik_runner_amd.csrc.ops import paired_order
    torch.manual_seed(H * 100 + D + ps)
    tables, n_pages = scatter_pages([s + n for s, n in zip(starts, q_lens)], ps, 2)
    ctx = FakeCtx(starts, q_lens, tables, ps)
    T, Q, K = sum(q_lens), H * D, Hk * D
    h = (torch.randn(T, E, device=DEV) * 0.5).to(DT[dt])
    w = (torch.randn(Q + 2 * K, E, device=DEV) * (0.2 if E < 500 else 0.05)).to(DT[dt])
    b = torch.randn(Q + 2 * K, device=DEV) * 0.3 if bias else None
    inv = (10000.0 ** (-torch.arange(rot // 2, dtype=torch.float64) * 2 / rot)).float().to(DEV) if rot else None
    paired = rot > 0 and not inter and rot % 16 == 0
    wp, bp = w, b
    if paired:
        order = paired_order(D, rot)
        assert sorted(order) == list(range(D))
        index = torch.tensor([hd * D + c for hd in range(H + Hk) for c in order] + list(range(Q + K, Q + 2 * K)), device=DEV)
        wp, bp = w.index_select(0, index), (b.index_select(0, index) if bias else None)
    proj = h.double() @ w.double().T + (b.double() if bias else 0)
    pos = ctx.positions.cpu()
    rotate = (lambda x: ref_rope(x, pos, inv.cpu(), inter)) if rot else (lambda x: x.double())
    want_q = rotate(proj[:, :Q].cpu().reshape(T, H, D))
    want_k = rotate(proj[:, Q:Q + K].cpu().reshape(T, Hk, D))
    want_v = proj[:, Q + K:].cpu().reshape(T, Hk, D)
    tol = 1e-5 if dt == "float32" else 6e-3
    results = []
    asked = []
    def step_table():                  # the step's cosines and sines, made once for all layers
        asked.append(1)
        return ops.rope_table(ctx.positions, inv, 1.0)
    for fuse in (True, False, "with the step's table"):
        kc = torch.full((n_pages, Hk, ps, D), float("nan"), device=DEV, dtype=DT[dt])
        vc = torch.full((n_pages, Hk, D, ps), float("nan"), device=DEV, dtype=DT[dt])
        ops.fuse_rope = bool(fuse)
        try:
            q = ops.project_rope_kv_write(h, ops.pack_weight(wp), bp, kc, vc, ctx.positions, ctx.req_of_token,
                                          ctx.block_table(0), inv, H, Hk, D, rot, inter, 1.0, ps, paired=paired,
                                          cs_table=step_table if fuse not in (True, False) and rot else None,
                                          variant=variant if fuse else 0)
        finally:
            ops.fuse_rope = True
        assert q.dtype == DT[dt] and rel(q.cpu().reshape(T, H, D), want_q) < tol
        written = torch.zeros(n_pages, ps, dtype=torch.bool)
        t = 0
        for r, (s, n) in enumerate(zip(starts, q_lens)):
            for p in range(s, s + n):
                page, off = tables[r][p // ps], p % ps
                assert rel(kc[page, :, off, :].cpu(), want_k[t]) < tol
                assert rel(vc[page, :, :, off].cpu(), want_v[t]) < tol
                written[page, off] = True
                t += 1
        assert torch.isnan(kc.float().cpu().permute(0, 2, 1, 3)[~written]).all()      # nothing else was touched
        assert torch.isnan(vc.float().cpu().permute(0, 3, 1, 2)[~written]).all()
        results.append((q.float().cpu(), torch.nan_to_num(kc.float().cpu()), torch.nan_to_num(vc.float().cpu())))
    if dt == "bfloat16":
        for one, two, three in zip(*results):   # the same sums and formulas: at most a rounding apart
            assert rel(one, two) < 4e-3
            assert torch.equal(one, three)      # a table made beforehand holds what the product would make itself
        # the table is asked for only where the tile kernel rotates (from 512 rows)
        assert len(asked) == (1 if rot and T >= 512 and (inter or paired) and D % 16 == 0 else 0)


def ref_attention(q, k_seq, v_seq, starts, q_lens, scale, window):
    """float64 attention per request; k_seq/v_seq[b]: [len, Hk, D] of the whole request."""
    outs = []
    t = 0
    for b, (s, n) in enumerate(zip(starts, q_lens)):
        k, v = k_seq[b].double(), v_seq[b].double()
        H, Hk = q.shape[1], k.shape[1]
        for i in range(n):
            p = s + i
            lo = max(0, p - window + 1) if window else 0
            qg = q[t].double().view(Hk, H // Hk, -1)            # query head h reads key/value head h // (H / Hk)
            sc = torch.einsum("kgd,tkd->kgt", qg, k[lo:p + 1]) * scale
            pr = torch.softmax(sc, dim=-1)
            outs.append(torch.einsum("kgt,tkd->kgd", pr, v[lo:p + 1]).reshape(H, -1))
            t += 1
    return torch.stack(outs)


def fill_cache(k_seq, v_seq, tables, n_pages, ps, dt):
    Hk, D = k_seq[0].shape[1:]
    kc = torch.full((n_pages, Hk, ps, D), float("nan"), dtype=dt)
    vc = torch.full((n_pages, Hk, D, ps), float("nan"), dtype=dt)
    for b, (k, v) in enumerate(zip(k_seq, v_seq)):
        full = k.shape[0] // ps                         # whole pages at once, the rest position by position
        if full:
            pages = torch.tensor(tables[b][:full], dtype=torch.long)
            kc[pages] = k[:full * ps].to(dt).view(full, ps, Hk, D).permute(0, 2, 1, 3)
            vc[pages] = v[:full * ps].to(dt).view(full, ps, Hk, D).permute(0, 2, 3, 1)
        for p in range(full * ps, k.shape[0]):
            kc[tables[b][p // ps], :, p % ps, :] = k[p].to(dt)
            vc[tables[b][p // ps], :, :, p % ps] = v[p].to(dt)
    return kc.to(DEV), vc.to(DEV)


ATTN_CASES = [
    # H, Hk, D, page, window, starts, q_lens
    (4, 2, 16, 16, None, [0, 5, 100], [33, 1, 1]),
    (3, 1, 32, 64, None, [0, 63, 64, 200], [70, 1, 2, 1]),
    (8, 2, 128, 16, None, [300, 0, 17], [1, 40, 5]),
    (6, 3, 48, 32, 24, [0, 90, 31], [50, 1, 3]),
    (4, 4, 64, 16, 7, [40, 0], [1, 20]),
    (5, 5, 80, 4, None, [10, 0], [3, 9]),          # small pages: the 32-bit kernel serves bfloat16 too
    (2, 1, 24, 8, 5, [0, 30], [12, 1]),            # head size no multiple of 16
    (32, 8, 128, 64, None, [2047, 1000], [1, 1]),  # decoding, long
    (5, 1, 80, 32, None, [300, 10], [1, 3]),       # decoding with a head size that is no power of two
    (4, 2, 256, 16, 600, [700, 3], [1, 2]),        # the largest head, small pages, a window that has given pages back
    (6, 2, 48, 64, None, [5000], [1]),             # more than 64 pages: the page numbers are fetched again on the way
    (64, 8, 128, 64, None, [900, 0, 130], [1, 70, 3]),   # 8 query heads a key/value head: 4 tokens x 8 heads in a 32-row block
    (32, 32, 128, 64, None, [700, 0, 64], [1, 150, 2]),  # one query head a key/value head, 32 of them: 32 tokens in a block
    (8, 2, 128, 64, None, [70001, 3], [1, 2]),           # a decoded token behind 70,000 keys (1,094 pages, 32 key ranges)
    (8, 2, 128, 64, None, [66000], [40]),                # a prompt portion behind 66,000 keys (128-row items cut into key ranges)
    (4, 1, 64, 32, 4096, [40000], [1]),                  # a window of 4,096 far into a long request
]


@pytest.mark.parametrize("case", [
    (8, 2, 128, 64, None, [37, 0, 900], [16, 40, 1]),      # 64-row and 160-row items of the workgroup kernel beside a decoded token
    (32, 8, 128, 64, None, [0], [300]),                     # a causal prompt: every wave of the workgroup kernel busy
    (6, 3, 64, 32, None, [100, 0], [33, 70]),
])
def test_attention_gives_the_same_bits_every_time(ops, case):
    """The same call eight times with other work between: the output is the same to the bit.  In the
    kernel that takes 128-row items two waves share a SIMD, and how their instructions interleave
    changes from run to run: a softmax reference read before the matrix unit had written it (an
    instruction the compiler does not schedule reading the accumulator) showed as last-bit differences
    between runs and nowhere else, since any reference gives the same quotient."""
    H, Hk, D, ps, window, starts, q_lens = case
    torch.manual_seed(7)
    lens = [s + n for s, n in zip(starts, q_lens)]
    tables, n_pages = scatter_pages(lens, ps, 5)
    ctx = FakeCtx(starts, q_lens, tables, ps)
    T = sum(q_lens)
    q = torch.randn(T, H * D).bfloat16().to(DEV)
    k_seq = [torch.randn(n, Hk, D).bfloat16() for n in lens]
    v_seq = [torch.randn(n, Hk, D).bfloat16() for n in lens]
    kc, vc = fill_cache(k_seq, v_seq, tables, n_pages, ps, torch.bfloat16)
    scale = 1 / math.sqrt(D)
    first = ops.attention(q, kc, vc, ctx, 0, H, Hk, D, ps, scale, window).clone()
    busy = torch.randn(1024, 1024, device=DEV)
    for i in range(8):
        if i % 2:
            busy = busy * 1.0001 + 1.0              # something else on the GPU between two calls
        again = ops.attention(q, kc, vc, ctx, 0, H, Hk, D, ps, scale, window)
        assert torch.equal(again.view(torch.int16), first.view(torch.int16)), f"call {i + 2} differs from the first"


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("case", ATTN_CASES)
def test_attention(ops, dt, case):
    H, Hk, D, ps, window, starts, q_lens = case
    torch.manual_seed(H * 100 + D)
    lens = [s + n for s, n in zip(starts, q_lens)]
    tables, n_pages = scatter_pages(lens, ps, D)
    ctx = FakeCtx(starts, q_lens, tables, ps)
    T = sum(q_lens)
    q = torch.randn(T, H, D).to(DT[dt])
    k_seq = [torch.randn(n, Hk, D).to(DT[dt]) for n in lens]
    v_seq = [torch.randn(n, Hk, D).to(DT[dt]) for n in lens]
    kc, vc = fill_cache(k_seq, v_seq, tables, n_pages, ps, DT[dt])
    scale = 1 / math.sqrt(D)
    want = ref_attention(q.float(), [k.float() for k in k_seq], [v.float() for v in v_seq], starts, q_lens, scale, window)
    got = ops.attention(q.to(DEV).reshape(T, H * D).contiguous(), kc, vc, ctx, 0, H, Hk, D, ps, scale, window)
    got = got.cpu().reshape(T, H, D)
    assert torch.isfinite(got.float()).all(), "read a slot no request owns"
    # 32-bit: 3e-6 of the largest output up to 4,096 keys; a row's sums over n keys are 32-bit running
    # sums whose rounding grows with the root of n (the cases behind 66,000 and 70,000 keys: x 4)
    tol32 = 3e-6 * max(1.0, math.sqrt(max(lens) / 4096))
    assert rel(got, want) < (tol32 if dt == "float32" else 1.2e-2)


def test_attention_items_longer_than_64_pages(ops):
    """A work item keeps 64 page numbers in its lanes and fetches the next 64 on the way: items
    that are not cut into key ranges (enough requests to fill the chip; a long portion left
    whole) walk through several such sets."""
    from xyntetik_runner_amd.engine.batch import plan_attention
    torch.manual_seed(11)
    # decoding: 32 requests x 8 key/value heads fill the chip, so nobody's 190 pages are cut
    H, Hk, D, ps = 8, 8, 16, 16
    starts = [2990 + 3 * i for i in range(32)]
    q_lens = [1] * 32
    assert all(it[4] == -1 for it in plan_attention(starts, q_lens, 1, None, Hk, ps)[1])
    # a portion of 70 tokens after 3000, left whole: 96 pages of 32
    for (H, Hk, D, ps, starts, q_lens, cta_tiles) in [(8, 8, 16, 16, starts, q_lens, None), (4, 2, 32, 32, [3000], [70], 1000)]:
        lens = [s + n for s, n in zip(starts, q_lens)]
        tables, n_pages = scatter_pages(lens, ps, 3)
        ctx = FakeCtx(starts, q_lens, tables, ps, cta_tiles=cta_tiles)
        T = sum(q_lens)
        q = torch.randn(T, H, D).bfloat16()
        k_seq = [torch.randn(n, Hk, D).bfloat16() for n in lens]
        v_seq = [torch.randn(n, Hk, D).bfloat16() for n in lens]
        # one key far back and one near the end stand out, in different sets of 64 pages
        for b, n in enumerate(lens):
            for far in (5, n - 40):
                k_seq[b][far] = (q[sum(q_lens[:b])].float().reshape(Hk, H // Hk, D)[:, 0] * 3).bfloat16()
        kc, vc = fill_cache(k_seq, v_seq, tables, n_pages, ps, torch.bfloat16)
        scale = 1 / math.sqrt(D)
        want = ref_attention(q.float(), [k.float() for k in k_seq], [v.float() for v in v_seq], starts, q_lens, scale, None)
        got = ops.attention(q.to(DEV).reshape(T, H * D).contiguous(), kc, vc, ctx, 0, H, Hk, D, ps, scale, None)
        got = got.cpu().reshape(T, H, D)
        assert torch.isfinite(got.float()).all()
        err = (got.double() - want).abs().amax(dim=(1, 2)) / want.abs().amax()
        assert err.max() < 1.2e-2, f"token {int(err.argmax())}: {float(err.max())}"


ATTN_WORKGROUP_CASES = [
    # H, Hk, D, page, window, starts, q_lens, most tiles per 128-row item (None: the engine's choice)
    (8, 2, 128, 64, None, [0], [300], None),
    (8, 2, 128, 64, None, [0], [300], 2),              # key ranges, merged afterwards
    (4, 1, 80, 32, None, [37, 0, 500], [130, 64, 1], 3),   # head size no power of two; a decoded token beside
    (6, 2, 256, 64, 100, [200], [150], None),          # window; the largest head
    (2, 2, 16, 32, None, [5], [70], 1),
    (5, 1, 64, 128, 33, [1000, 3], [90, 40], 4),       # five heads a group: rows of a token straddle waves
    (3, 3, 48, 32, 9, [60], [200], None),              # a window shorter than a tile
    (4, 2, 128, 32, None, [37, 0], [200, 96], None),   # a tile a page: whole tiles come from bases all lanes share
    (4, 4, 64, 32, 50, [300, 31], [100, 70], 2),       # the same with a window and key ranges
]


@pytest.mark.parametrize("case", ATTN_WORKGROUP_CASES)
def test_attention_long_portions(ops, case):
    """Portions of 64 rows and more go to the kernel that shares key and value tiles in a workgroup."""
    H, Hk, D, ps, window, starts, q_lens, cta_tiles = case
    torch.manual_seed(H * 100 + D)
    lens = [s + n for s, n in zip(starts, q_lens)]
    tables, n_pages = scatter_pages(lens, ps, D)
    ctx = FakeCtx(starts, q_lens, tables, ps, cta_tiles=cta_tiles)
    plan = ctx.attention_plan(0, H // Hk, window, Hk, ps)
    assert plan.n_cta_items > 0
    T = sum(q_lens)
    q = torch.randn(T, H, D).bfloat16()
    k_seq = [torch.randn(n, Hk, D).bfloat16() for n in lens]
    v_seq = [torch.randn(n, Hk, D).bfloat16() for n in lens]
    kc, vc = fill_cache(k_seq, v_seq, tables, n_pages, ps, torch.bfloat16)
    scale = 1 / math.sqrt(D)
    want = ref_attention(q.float(), [k.float() for k in k_seq], [v.float() for v in v_seq], starts, q_lens, scale, window)
    got = ops.attention(q.to(DEV).reshape(T, H * D).contiguous(), kc, vc, ctx, 0, H, Hk, D, ps, scale, window)
    got = got.cpu().reshape(T, H, D)
    assert torch.isfinite(got.float()).all(), "read a slot no request owns"
    # row by row, so that a wrong row among hundreds shows
    err = (got.double() - want).abs().amax(dim=(1, 2)) / want.abs().amax()
    assert err.max() < 1.2e-2, f"token {int(err.argmax())}: {float(err.max())}"


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("far", [0, 15, 16, 31, 32, 63, 64, 255, 256, 700, 1023])
def test_attention_finds_one_far_key(ops, dt, far):
    """One key among a thousand is made to stand out: the output must be its value row.
    The key sits at the first slot, at page and tile edges, and at the last position."""
    H, Hk, D, ps = 4, 2, 64, 16
    n = 1024
    torch.manual_seed(far)
    tables, n_pages = scatter_pages([n], ps, far)
    k = torch.randn(n, Hk, D) * 0.1
    v = torch.randn(n, Hk, D)
    q = torch.randn(1, H, D) * 0.1
    q[0, :, :] += 4.0
    k[far, :, :] += 4.0                      # score of `far` stands out by ~ 4*4*64/8
    kc, vc = fill_cache([k], [v], tables, n_pages, ps, DT[dt])
    ctx = FakeCtx([n - 1], [1], tables, ps)
    got = ops.attention(q.to(DT[dt]).to(DEV).reshape(1, H * D), kc, vc, ctx, 0, H, Hk, D, ps, 1 / math.sqrt(D))
    want = v.to(DT[dt]).float()[far].repeat_interleave(H // Hk, dim=0)
    assert rel(got.cpu().reshape(H, D), want) < (1e-5 if dt == "float32" else 1e-2)


@pytest.mark.parametrize("start,far", [(0, 3), (32, 5), (32, 40), (64, 10), (64, 50), (64, 70), (224, 100), (224, 140),
                                        (230, 127), (230, 128), (2000, 1023), (2000, 1024), (2000, 1999)])
def test_attention_two_wave_sets_share_an_item(ops, start, far):
    """A 128-row item's tiles go half to one set of waves and half to another, whose results are
    combined at the end.  One key is made to stand out, in the first half, in the second, at the
    edge between them, with one to 64 tiles an item (the second set has nothing to do with one
    tile) and a last tile that is not full: every row that may see the key must return its value."""
    H, Hk, D, ps, n_new = 4, 1, 128, 64, 38          # 152 rows: one item of 128 rows and one of 24
    n = start + n_new
    torch.manual_seed(start * 7 + far)
    tables, n_pages = scatter_pages([n], ps, far)
    k = torch.randn(n, Hk, D) * 0.1
    v = torch.randn(n, Hk, D)
    q = torch.randn(n_new, H, D) * 0.1 + 4.0
    k[far] += 4.0
    kc, vc = fill_cache([k], [v], tables, n_pages, ps, torch.bfloat16)
    ctx = FakeCtx([start], [n_new], tables, ps, cta_tiles=1000)
    plan = ctx.attention_plan(0, H // Hk, None, Hk, ps)
    assert plan.n_cta_items == 2 and plan.n_jobs == 0
    got = ops.attention(q.bfloat16().to(DEV).reshape(n_new, H * D), kc, vc, ctx, 0, H, Hk, D, ps, 1 / math.sqrt(D))
    got = got.cpu().reshape(n_new, H, D).float()
    assert torch.isfinite(got).all()
    want = ref_attention(q.bfloat16().float(), [k.bfloat16().float()], [v.bfloat16().float()], [start], [n_new], 1 / math.sqrt(D), None)
    err = (got.double() - want).abs().amax(dim=(1, 2)) / want.abs().amax()
    assert err.max() < 1.2e-2, f"token {int(err.argmax())}: {float(err.max())}"
    sees = [t for t in range(n_new) if start + t >= far]
    assert sees and rel(got[sees], v.bfloat16().float()[far].expand(len(sees), H, D)) < 1e-2


@pytest.mark.parametrize("H,Hk,D,ps,window,start", [(1, 1, 128, 64, None, 1111), (4, 1, 128, 32, None, 1111), (2, 2, 64, 64, None, 600),
                                                      (1, 1, 128, 64, 700, 1111), (2, 1, 256, 64, None, 500)])
def test_attention_every_token_has_a_far_key_of_its_own(ops, H, Hk, D, ps, window, start):
    """A step of the workgroup kernel works on three tiles at once (the scores of one, the softmax of
    the one before, the value product of the one before that) out of four places of a ring in LDS.  Here
    every token of a 160-token portion has one key that stands out, and these keys are spread over all the
    tiles the token may see (with a window: over the tiles inside it): whichever tile, place of the ring,
    step of the loop or set of waves a key falls to, its token must come back with that key's value."""
    n_new = 160
    n = start + n_new
    g = torch.Generator().manual_seed(D + ps + start)
    u = (torch.randint(0, 2, (n_new, D), generator=g).float() * 2 - 1) * 1.5      # q . k = 2.25 D for a token's own key
    span = window if window else start
    far = [start + t - (t * 37) % span if window else (t * 37) % start for t in range(n_new)]
    assert len(set(p // 32 for p in far)) >= min(20, span // 32)      # many different tiles
    k = torch.randn(n, Hk, D, generator=g) * 0.1
    v = torch.randn(n, Hk, D, generator=g)
    q = u[:, None, :].expand(n_new, H, D).contiguous()
    for t, p in enumerate(far):
        k[p] = u[t]
    tables, n_pages = scatter_pages([n], ps, 5)
    kc, vc = fill_cache([k], [v], tables, n_pages, ps, torch.bfloat16)
    ctx = FakeCtx([start], [n_new], tables, ps, cta_tiles=1000)
    plan = ctx.attention_plan(0, H // Hk, window, Hk, ps)
    assert plan.n_cta_items >= 1 and plan.n_jobs == 0
    scale = 1 / math.sqrt(D)
    got = ops.attention(q.bfloat16().to(DEV).reshape(n_new, H * D), kc, vc, ctx, 0, H, Hk, D, ps, scale, window)
    got = got.cpu().reshape(n_new, H, D).float()
    want = ref_attention(q.bfloat16().float(), [k.bfloat16().float()], [v.bfloat16().float()], [start], [n_new], scale, window)
    err = (got.double() - want).abs().amax(dim=(1, 2)) / want.abs().amax()
    assert err.max() < 1.2e-2, f"token {int(err.argmax())} (its key at {far[int(err.argmax())]}): {float(err.max())}"
    own = torch.stack([v.bfloat16().float()[p] for p in far]).repeat_interleave(H // Hk, dim=1)
    assert rel(got, own) < 2e-2


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
def test_attention_window_edge(ops, dt):
    """The key just outside the window is made huge: it must not be seen; the one just inside must."""
    H, Hk, D, ps, window = 2, 1, 32, 16, 20
    n = 100
    tables, n_pages = scatter_pages([n], ps, 3)
    k = torch.randn(n, Hk, D) * 0.1
    v = torch.randn(n, Hk, D)
    q = torch.full((1, H, D), 2.0)
    outside, inside = n - 1 - window, n - window
    k[outside] += 50.0
    kc, vc = fill_cache([k], [v], tables, n_pages, ps, DT[dt])
    ctx = FakeCtx([n - 1], [1], tables, ps)
    run = lambda kc_: ops.attention(q.to(DT[dt]).to(DEV).reshape(1, H * D), kc_, vc, ctx, 0, H, Hk, D, ps, 1 / math.sqrt(D), window).cpu().reshape(H, D)
    got = run(kc)
    assert rel(got, v.to(DT[dt]).float()[outside].expand(H, D)) > 0.1          # the outside key is not what we got
    want = ref_attention(q.to(DT[dt]).float(), [k.to(DT[dt]).float()], [v.to(DT[dt]).float()], [n - 1], [1], 1 / math.sqrt(D), window)[0]
    assert rel(got, want) < (3e-6 if dt == "float32" else 1.2e-2)
    k2 = k.clone(); k2[inside] += 50.0
    kc2, _ = fill_cache([k2], [v], tables, n_pages, ps, DT[dt])
    assert rel(run(kc2), v.to(DT[dt]).float()[inside].expand(H, D)) < (1e-5 if dt == "float32" else 1e-2)


def test_attention_plan_covers_every_key_once():
    from xyntetik_runner_amd.engine.batch import plan_attention
    for starts, q_lens, G, window, Hk, cta_tiles in [
            ([0, 100, 4000], [70, 1, 1], 4, None, 8, None), ([5000], [1], 4, None, 8, None),
            ([0], [2048], 4, None, 8, None), ([300, 2], [1, 9], 2, 50, 1, None),
            ([10, 0], [333, 15], 3, 40, 2, 2), ([0], [100], 5, None, 1, 1)]:
        cta_items, items, jobs, n_slots = plan_attention(starts, q_lens, G, window, Hk, 64, cta_tiles)
        used = []
        for rows, waves, some in ((128, 4, cta_items), (32, 1, items)):
            by_block = {}
            for b, row0, k0, k1, slot, q0, q_len, start in some:
                assert k0 % 32 == 0 and k0 < k1
                assert q0 == sum(q_lens[:b]) and q_len == q_lens[b] and start == starts[b]
                by_block.setdefault((b, row0), []).append((k0, k1, slot))
            for (b, row0), parts in by_block.items():
                parts.sort()
                n = q_lens[b]
                hi = starts[b] + min(n - 1, (row0 + rows - 1) // G) + 1
                lo = 0 if not window else max(0, starts[b] + row0 // G - window + 1)
                assert parts[0][0] <= lo and parts[-1][1] == hi
                assert all(a[1] == c[0] for a, c in zip(parts, parts[1:]))
                assert (len(parts) == 1) == (parts[0][2] == -1)
                if len(parts) > 1:
                    for w in range(waves):              # every 32-row block that exists is merged from its slots
                        if row0 + 32 * w < n * G:
                            assert (b, row0 + 32 * w, parts[0][2] + w, len(parts), waves, sum(q_lens[:b]), q_lens[b]) in jobs
                    used += [p[2] + w for p in parts for w in range(waves)]
        # a row belongs to one kind of item only
        assert not {(b, r // 128) for b, r, *_ in cta_items} & {(b, r // 128) for b, r, *_ in items}
        assert sorted(used) == list(range(n_slots))
        assert sum(j[3] for j in jobs if j[1] // 32 * 32 == j[1]) <= n_slots
