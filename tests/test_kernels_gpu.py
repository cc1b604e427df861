"""Each kernel alone against a plain float64/float32 torch computation of the same op,
at sizes other than the engine's (widths that are no power of two, odd row counts)."""

from __future__ import annotations

import math

import pytest
import torch

from tests.plain import llama as plain
from tests.plain import sampling as plain_sampling

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module")
def ops():
    from kvcore_amd.ops import library

    library.load()
    return library


def tol(dtype):
    return dict(atol=2e-6, rtol=2e-6) if dtype == torch.float32 else dict(atol=1e-2, rtol=1e-2)


def rnd(*shape, dtype=torch.float32, scale=1.0, seed=0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


@pytest.mark.parametrize("dtype", DTYPES)
def test_embed(ops, dtype):
    V, H = 37, 100
    table = rnd(V, H, dtype=dtype)
    ids = torch.tensor([0, 36, 5, 5, 40, -1], dtype=torch.int32, device=DEV)
    out = torch.zeros(6, H, device=DEV)
    ops.embed(out, table, ids)
    assert torch.equal(out[:4], table.float()[ids[:4].long()])
    assert torch.isnan(out[4:]).all()  # an id outside the table is loud, not a stray read
    ops.embed(out, table, ids, 2.5)
    assert torch.equal(out[:4], table.float()[ids[:4].long()] * 2.5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H", [96, 200, 4100, 4096, 12296])
def test_add_rmsnorm(ops, dtype, H):
    T, eps = 5, 1e-5
    residual = rnd(T, H, seed=1)
    delta = rnd(T, H, dtype=dtype, seed=2)
    w = 1 + 0.1 * rnd(H, seed=3)
    want_res = residual.double() + delta.double()
    want = plain.rms_norm(want_res, w.double(), eps)
    out = torch.empty(T, H, dtype=dtype, device=DEV)
    res = residual.clone()
    ops.add_rmsnorm(out, res, delta, w, eps)
    assert torch.allclose(res.double(), want_res, atol=1e-6)  # the sum stays float32
    assert torch.allclose(out.double(), want, **tol(dtype))
    res2 = residual.clone()
    ops.add_rmsnorm(out, res2, None, w, eps)
    assert torch.equal(res2, residual)
    assert torch.allclose(out.double(), plain.rms_norm(residual.double(), w.double(), eps), **tol(dtype))
    ops.residual_add(res2, delta)
    assert torch.allclose(res2.double(), want_res, atol=1e-6)


@pytest.mark.parametrize("dtype", DTYPES)
def test_rmsnorm_on_strided_rows(ops, dtype):
    big = rnd(7, 300, dtype=dtype)
    x = big[:, 20:116]
    w = 1 + 0.1 * rnd(96, seed=4)
    out = torch.empty(7, 96, dtype=dtype, device=DEV)
    ops.rmsnorm(out, x, w, 1e-6)
    assert torch.allclose(out.double(), plain.rms_norm(x.double(), w.double(), 1e-6), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
def test_silu_mul(ops, dtype):
    gu = rnd(9, 2 * 177, dtype=dtype, scale=3.0)
    out = torch.empty(9, 177, dtype=dtype, device=DEV)
    ops.silu_mul(out, gu)
    assert torch.allclose(out.double(), plain.silu_and_mul(gu.double()), **tol(dtype))


def test_gather_rows_and_to_float(ops):
    src = rnd(10, 50)
    rows = torch.tensor([9, 0, 3, 3], dtype=torch.int32, device=DEV)
    out = torch.empty(4, 50, dtype=torch.bfloat16, device=DEV)
    ops.gather_rows(out, src, rows)
    assert torch.equal(out, src[rows.long()].to(torch.bfloat16))
    back = torch.empty(4, 50, device=DEV)
    ops.to_float(back, out)
    assert torch.equal(back, out.float())


@pytest.mark.parametrize("M,N,K", [(1, 130, 100), (3, 64, 16), (70, 257, 333), (128, 96, 96)])
def test_gemm_f32_is_true_float32_and_does_not_depend_on_the_batch(ops, M, N, K):
    a, w, b = rnd(M, K, seed=1), rnd(N, K, seed=2), rnd(N, seed=3)
    out = torch.empty(M, N, device=DEV)
    ops.gemm_f32(out, a, w, b)
    want = a.double() @ w.double().T + b.double()
    # float32 products and sums: error grows like sqrt(K) * 2^-24 of the summed magnitudes
    bound = 4 * math.sqrt(K) * 2 ** -24 * (a.double().abs() @ w.double().abs().T + b.double().abs())
    assert ((out.double() - want).abs() <= bound + 1e-7).all()
    # a row alone gives the same bits as inside the batch
    single = torch.empty(1, N, device=DEV)
    for i in {0, M // 2, M - 1}:
        ops.gemm_f32(single, a[i:i + 1].contiguous(), w, b)
        assert torch.equal(single[0], out[i])
    # strided output and input rows
    wide_in = torch.zeros(M, K + 7, device=DEV)
    wide_in[:, :K] = a
    wide_out = torch.zeros(M, N + 5, device=DEV)
    ops.gemm_f32(wide_out[:, :N], wide_in[:, :K], w, None)
    assert torch.equal(wide_out[:, :N], out - b) or torch.allclose(wide_out[:, :N], out - b, atol=1e-5)
    assert torch.all(wide_out[:, N:] == 0)


@pytest.mark.parametrize("M,N,K", [(1, 16, 64), (5, 100, 200), (8, 4096, 4096), (16, 130, 1032),
                                   (17, 6144, 512), (33, 48, 14336), (64, 1000, 2048),
                                   # the longest sum and the widest output of the 70B shape
                                   (8, 8192, 28672), (12, 57344, 8192)])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
def test_gemm_skinny_bf16(ops, M, N, K, out_dtype):
    a = rnd(M, K, dtype=torch.bfloat16, seed=1)
    w = rnd(N, K, dtype=torch.bfloat16, seed=2, scale=0.05)
    bias = rnd(N, dtype=torch.bfloat16, seed=3)
    out = torch.full((M, N), float("nan"), dtype=out_dtype, device=DEV)
    ops.gemm_skinny_bf16(out, a, w, bias)
    want = a.double() @ w.double().T + bias.double()
    mag = a.double().abs() @ w.double().abs().T + bias.double().abs()
    err = (out.double() - want).abs()
    # float32 sums of exact bfloat16 products; a bfloat16 result adds one rounding of 2^-9
    bound = 8 * math.sqrt(K) * 2 ** -24 * mag + 1e-6
    if out_dtype == torch.bfloat16:
        bound = bound + want.abs() * 2 ** -8
    assert (err <= bound).all(), float((err / bound).max())
    # a row alone, or in another place of the batch, gives the same bits
    single = torch.empty(1, N, dtype=out_dtype, device=DEV)
    for i in {0, M // 2, M - 1}:
        ops.gemm_skinny_bf16(single, a[i:i + 1].contiguous(), w, bias)
        assert torch.equal(single[0], out[i])
    # strided rows in and out, no bias
    wide_in = torch.zeros(M, K + 8, dtype=torch.bfloat16, device=DEV)
    wide_in[:, :K] = a
    wide_out = torch.zeros(M, N + 3, dtype=out_dtype, device=DEV)
    ops.gemm_skinny_bf16(wide_out[:, :N], wide_in[:, :K], w, None)
    ref = torch.empty(M, N, dtype=out_dtype, device=DEV)
    ops.gemm_skinny_bf16(ref, a, w, None)
    assert torch.equal(wide_out[:, :N], ref) and torch.all(wide_out[:, N:] == 0)


@pytest.mark.parametrize("M,N,K", [(17, 200, 512), (33, 64, 1024), (48, 1000, 1536), (64, 4104, 1024),
                                   (5, 72, 512), (64, 16400, 512),
                                   # more than four tiles of 16 rows: five and six run as six, seven and eight as eight
                                   (65, 200, 1024), (81, 4104, 512), (96, 1000, 1536), (100, 16400, 512),
                                   (128, 4096, 4096), (113, 72, 512),
                                   # nine to twelve tiles run as twelve
                                   (129, 200, 512), (192, 4096, 4096), (150, 1000, 1536), (192, 16400, 512), (177, 72, 1024),
                                   # the longest sum and the widest output of the 70B shape
                                   (40, 8192, 28672), (24, 57344, 8192), (128, 8192, 28672)])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_gemm_mid_bf16(ops, M, N, K, out_dtype):
    """The product for a few dozen rows, whose waves share the rows through LDS: at once, and
    cut along K into partial sums that a second kernel adds up."""
    a = rnd(M, K, dtype=torch.bfloat16, seed=1)
    w = rnd(N, K, dtype=torch.bfloat16, seed=2, scale=0.05)
    bias = rnd(N, dtype=torch.bfloat16, seed=3)
    want = a.double() @ w.double().T + bias.double()
    mag = a.double().abs() @ w.double().abs().T + bias.double().abs()
    bound = 8 * math.sqrt(K) * 2 ** -24 * mag + 1e-6
    if out_dtype == torch.bfloat16:
        bound = bound + want.abs() * 2 ** -8
    slices = ops.mid_slices(N, K)
    assert 1 <= slices <= ops.mid_slices_bound(N)
    partial = torch.full((slices * M * N,), float("nan"), device=DEV)
    outs = {}
    for mode in (0, 3):
        out = torch.full((M, N), float("nan"), dtype=out_dtype, device=DEV)
        ops.gemm_mid(out, a, w, bias, mode=mode, partial=partial if mode == 3 else None)
        err = (out.double() - want).abs()
        assert (err <= bound).all(), (mode, float((err / bound).max()))
        outs[mode] = out
    # the partial sums alone: their sum in slice order is what mode 3 stored
    ops.gemm_mid(None, a, w, mode=2, partial=partial)
    total = partial[: slices * M * N].view(slices, M, N)[0].clone()
    for s_ in range(1, slices):
        total += partial[: slices * M * N].view(slices, M, N)[s_]
    assert torch.equal((total + bias.float()).to(out_dtype), outs[3])
    # fewer rows of the same batch give the same bits: the launch depends on N and K alone
    few = min(M, 18)
    out_few = torch.empty(few, N, dtype=out_dtype, device=DEV)
    ops.gemm_mid(out_few, a[:few].contiguous(), w, bias, mode=0)
    assert torch.equal(out_few, outs[0][:few])
    # strided rows in and out
    wide_in = torch.zeros(M, K + 8, dtype=torch.bfloat16, device=DEV)
    wide_in[:, :K] = a
    wide_out = torch.zeros(M, N + 3, dtype=out_dtype, device=DEV)
    ops.gemm_mid(wide_out[:, :N], wide_in[:, :K], w, bias, mode=0)
    assert torch.equal(wide_out[:, :N], outs[0]) and torch.all(wide_out[:, N:] == 0)


@pytest.mark.parametrize("M,I,K", [(17, 72, 512), (40, 1000, 1024), (64, 8200, 512), (40, 28672, 8192),
                                   (72, 1000, 1024), (96, 8200, 512), (128, 14336, 4096), (127, 72, 512),
                                   (130, 1000, 512), (160, 8200, 1024), (192, 14336, 4096), (191, 72, 512)])
@pytest.mark.parametrize("with_bias", [False, True])
def test_gemm_mid_silu_mul(ops, M, I, K, with_bias):
    x = rnd(M, K, dtype=torch.bfloat16, seed=1)
    w = rnd(2 * I, K, dtype=torch.bfloat16, seed=2, scale=0.1)
    bias = rnd(2 * I, dtype=torch.bfloat16, seed=3) if with_bias else None
    out = torch.full((M, I), float("nan"), dtype=torch.bfloat16, device=DEV)
    if ops.mid_rows_ok(M, False, ops.MID_ROWS_GATED):
        ops.linear_silu_mul(out, x, w, bias, lambda: pytest.fail("the one-kernel form should have run"))
    else:  # fewer or more rows take the one-kernel form only with a packed copy of the weights (tested below)
        ops.gemm_mid(out, x, w, bias, mode=1)
    # both factors rounded to bfloat16 first, as the two-kernel form stores them (the two
    # forms start their walks along K at different places, so not the same bits)
    gu = torch.empty(M, 2 * I, dtype=torch.bfloat16, device=DEV)
    ops.gemm_mid(gu, x, w, bias, mode=0)
    want = torch.empty(M, I, dtype=torch.bfloat16, device=DEV)
    ops.silu_mul(want, gu)
    assert torch.allclose(out.float(), want.float(), atol=2e-2, rtol=2e-2)
    exact = x.double() @ w.double().T + (bias.double() if with_bias else 0)
    formula = torch.nn.functional.silu(exact[:, :I]) * exact[:, I:]
    assert torch.allclose(out.double(), formula, atol=3e-2, rtol=3e-2)


def test_beyond_64_rows_the_kernel_for_a_few_dozen_rows_runs_where_it_was_measured_faster(ops, monkeypatch):
    """Packed weights: the gated product from 17 to 128 rows, the products cut along K up to
    192; weights read row by row only from 33 to 64 rows, the vendor's product has the rest."""
    ran = []
    real_mid, real_mm = ops.gemm_mid, torch.mm
    monkeypatch.setattr(ops, "gemm_mid", lambda *a, **kw: (ran.append("mid"), real_mid(*a, **kw))[1])
    monkeypatch.setattr(torch, "mm", lambda *a, **kw: (ran.append("vendor"), real_mm(*a, **kw))[1])
    I, K, H = 4096, 512, 512
    w_gate_up = (rnd(2 * I, K, dtype=torch.bfloat16, seed=2) * 0.1).contiguous()
    w_down = (rnd(H, I, dtype=torch.bfloat16, seed=3) * 0.1).contiguous()
    for packed in (False, True):
        if packed:
            ops.pack_weight(w_gate_up)
            ops.pack_weight(w_down)
        for M, gated_ours, sliced_ours in ((24, packed, packed), (33, True, True), (64, True, True), (96, packed, packed), (128, packed, packed), (144, False, packed),
                                           (192, False, packed), (200, False, False)):
            x = rnd(M, K, dtype=torch.bfloat16, seed=1)
            h = torch.empty(M, I, dtype=torch.bfloat16, device=DEV)
            scratch = torch.empty(M, 2 * I, dtype=torch.bfloat16, device=DEV)
            ran.clear()
            ops.linear_silu_mul(h, x, w_gate_up, None, lambda: scratch)
            assert ran == (["mid"] if gated_ours else ["vendor"]), (packed, M, ran)  # (8192 x 512 is no matrix for the few-row kernel at 24 rows)
            want = torch.nn.functional.silu(x.double() @ w_gate_up[:I].double().T) * (x.double() @ w_gate_up[I:].double().T)
            assert torch.allclose(h.double(), want, atol=3e-2, rtol=3e-2)
            if M > ops.MID_ROWS:
                continue  # no sink beyond the kernel's row limit: the block adds and normalises itself
            residual = rnd(M, H, seed=5)
            r0 = residual.clone()
            sink = ops.ResidualSink(residual, torch.ones(H, device=DEV), 1e-5, torch.empty(M, H, dtype=torch.bfloat16, device=DEV),
                                    None, torch.empty(ops.mid_slices_bound(H) * ops.MID_ROWS * H, device=DEV))
            ran.clear()
            ops.linear(sink, h, w_down)
            # (a small matrix at up to 32 rows goes to the few-row kernel instead of the vendor's)
            assert ran == (["mid"] if sliced_ours else ([] if M <= 32 else ["vendor"])), (packed, M, ran)
            assert torch.allclose((residual - r0).double(), h.double() @ w_down.double().T, atol=5e-2, rtol=3e-2)


def test_gemm_mid_refuses_what_it_does_not_take(ops):
    a = rnd(20, 520, dtype=torch.bfloat16)
    w = rnd(64, 520, dtype=torch.bfloat16)
    with pytest.raises(ops.KernelError, match="multiple of 512"):
        ops.gemm_mid(torch.empty(20, 64, dtype=torch.bfloat16, device=DEV), a, w)
    a = rnd(193, 512, dtype=torch.bfloat16)
    w = rnd(64, 512, dtype=torch.bfloat16)
    with pytest.raises(ops.KernelError, match="1 to 192 rows"):
        ops.gemm_mid(torch.empty(193, 64, dtype=torch.bfloat16, device=DEV), a, w)


@pytest.mark.parametrize("T,H,slices,with_bias", [(17, 64, 1, False), (40, 1000, 3, True), (64, 4096, 4, False),
                                                   (33, 16384, 2, True)])
def test_add_slices_rmsnorm(ops, T, H, slices, with_bias):
    residual = rnd(T, H, seed=1)
    partial = rnd(slices, T, H, seed=2)
    bias = rnd(H, dtype=torch.bfloat16, seed=3) if with_bias else None
    weight = rnd(H, seed=4) + 1.0
    eps = 1e-5
    r0 = residual.clone()
    out = torch.full((T, H), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.add_slices_rmsnorm(out, residual, partial, slices, bias, weight, eps)
    delta = partial[0].clone()
    for s_ in range(1, slices):
        delta += partial[s_]
    if with_bias:
        delta += bias.float()
    assert torch.equal(residual, r0 + delta)  # slice order, then into the residual
    r = residual.double()
    want = r * torch.rsqrt((r * r).mean(dim=1, keepdim=True) + eps) * weight.double()
    assert torch.allclose(out.double(), want, atol=1e-2, rtol=1e-2)


def test_sink_for_a_few_dozen_rows_finishes_the_norm(ops):
    """``linear`` into a sink with 17 to 64 rows: partial sums and one kernel that adds and
    normalises; a width the weight-streaming kernel does not take goes through the vendor
    product and gives the same rows beyond rounding."""
    for M, N, K in ((20, 256, 1024), (64, 4096, 512), (33, 200, 520)):
        x = rnd(M, K, dtype=torch.bfloat16, seed=1)
        w = rnd(N, K, dtype=torch.bfloat16, seed=2, scale=0.05)
        gain = rnd(N, seed=3) + 1.0
        residual = rnd(M, N, seed=4)
        r0 = residual.clone()
        rows = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
        work = torch.empty(ops.mid_slices_bound(N) * ops.MID_ROWS, N, device=DEV)
        got = ops.linear(ops.ResidualSink(residual, gain, 1e-5, rows, None, work), x, w)
        assert isinstance(got, ops.NormedRows) and got.data is rows
        r = r0.double() + x.double() @ w.double().T
        assert torch.allclose(residual.double(), r, atol=2e-2, rtol=1e-2)
        want = r * torch.rsqrt((r * r).mean(dim=1, keepdim=True) + 1e-5) * gain.double()
        assert torch.allclose(rows.double(), want, atol=3e-2, rtol=2e-2)


@pytest.mark.parametrize("M,I,K", [(1, 16, 64), (5, 100, 200), (8, 2072, 512), (16, 88, 1032),
                                   (17, 176, 80), (64, 40, 256)])
@pytest.mark.parametrize("with_bias", [False, True])
def test_linear_silu_mul(ops, M, I, K, with_bias):
    """The one-kernel form matches the formula, and gives the bits of the two-kernel form
    (product stored in bfloat16, then the activation) where both split K the same way."""
    x = rnd(M, K, dtype=torch.bfloat16, seed=1)
    w = rnd(2 * I, K, dtype=torch.bfloat16, seed=2, scale=0.1)
    bias = rnd(2 * I, dtype=torch.bfloat16, seed=3) if with_bias else None
    out = torch.full((M, I), float("nan"), dtype=torch.bfloat16, device=DEV)
    used_scratch = []

    def scratch():
        used_scratch.append(True)
        return torch.empty(M, 2 * I, dtype=torch.bfloat16, device=DEV)

    ops.linear_silu_mul(out, x, w, bias, scratch)
    assert bool(used_scratch) == (M > 16)
    gate_up = torch.empty(M, 2 * I, dtype=torch.bfloat16, device=DEV)
    ops.gemm_skinny_bf16(gate_up, x, w, bias)
    two = torch.empty_like(out)
    ops.silu_mul(two, gate_up)
    if M <= 16 and 2 * I > 4096:
        assert torch.equal(out, two)
    gu = x.double() @ w.double().T + (bias.double() if with_bias else 0.0)
    want = plain.silu_and_mul(gu)
    assert torch.allclose(out.double(), want, atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("M,N,K", [(1, 16, 64), (3, 64, 128), (8, 4096, 4096), (8, 144, 1088), (16, 1024, 512),
                                   (40, 96, 192)])
def test_packed_weights_give_the_same_bits(ops, M, N, K):
    """``pack_weight`` stores the matrix in the order the few-row products read it; they must
    give, bit for bit, what they give from the plain matrix: plain, gated, with the norms
    folded in, with bias."""
    x = rnd(M, K, dtype=torch.bfloat16, seed=1)
    w = (rnd(N, K, dtype=torch.bfloat16, seed=2) * 0.1).contiguous()
    bias = rnd(N, dtype=torch.bfloat16, seed=3)
    ss = (rnd(M, 4, seed=5).abs() + 0.5).contiguous()
    gain = rnd(N, seed=6).abs() + 0.5
    plain_out = {}
    for packed in (False, True):
        if packed:
            tiles = ops.pack_weight(w)
            # element (n, k) sits at ((n / 16) * (K / 32) + k / 32) * 512 + (n % 16) * 32 + k % 32
            want = w.view(N // 16, 16, K // 32, 32).permute(0, 2, 1, 3).contiguous().view(N, K)
            assert torch.equal(tiles.view(torch.int16), want.view(torch.int16)) and w.kvc_packed is tiles
        outs = []
        for out_dtype in (torch.bfloat16, torch.float32):
            out = torch.empty(M, N, dtype=out_dtype, device=DEV)
            ops.gemm_skinny_bf16(out, x, w, bias)
            outs.append(out)
        if N % 32 == 0:  # gated: the first half of the rows is the gate, the second the up factor
            out = torch.empty(M, N // 2, dtype=torch.bfloat16, device=DEV)
            ops.linear_silu_mul(out, x, w, bias, lambda: torch.empty(M, N, dtype=torch.bfloat16, device=DEV))
            outs.append(out)
        if M <= 16:
            # the fold: scaled rows in, residual sink out
            rows = ops.ScaledRows(x, ss, K, 1e-5)
            residual = rnd(M, N, dtype=torch.float32, seed=4)
            sink = ops.ResidualSink(residual=residual, gain=gain, eps=1e-5,
                                    out=torch.empty(M, N, dtype=torch.bfloat16, device=DEV),
                                    ss_parts=torch.empty(M * ops.skinny_blocks(N, K), device=DEV))
            got = ops.linear(sink, rows, w, bias)
            outs += [sink.out.clone(), residual.clone(), got.ss_parts.clone()]
        if packed:
            assert len(outs) == len(plain_out["outs"])
            for a, b in zip(outs, plain_out["outs"]):
                assert torch.equal(a.view(torch.int16 if a.dtype == torch.bfloat16 else torch.int32),
                                   b.view(torch.int16 if b.dtype == torch.bfloat16 else torch.int32))
        else:
            plain_out["outs"] = outs
    ref = x.float() @ w.float().t() + bias.float()
    assert torch.allclose(plain_out["outs"][1], ref, atol=2e-2, rtol=2e-2)
    with pytest.raises(ops.KernelError, match="pack_weight"):
        ops.pack_weight(w[:, :32])


@pytest.mark.parametrize("M,N,K", [(17, 64, 512), (40, 1008, 1024), (64, 4096, 1536)])
def test_packed_weights_give_the_same_bits_at_a_few_dozen_rows(ops, M, N, K):
    x = rnd(M, K, dtype=torch.bfloat16, seed=1)
    w = (rnd(N, K, dtype=torch.bfloat16, seed=2) * 0.1).contiguous()
    bias = rnd(N, dtype=torch.bfloat16, seed=3)
    results = []
    for packed in (False, True):
        if packed:
            ops.pack_weight(w)
        outs = []
        for mode in (0, 3):
            for out_dtype in (torch.bfloat16, torch.float32):
                out = torch.empty(M, N, dtype=out_dtype, device=DEV)
                part = torch.empty(ops.mid_slices(N, K) * M * N, device=DEV)
                ops.gemm_mid(out, x, w, bias, mode=mode, partial=part if mode == 3 else None)
                outs.append(out)
        part = torch.zeros(ops.mid_slices(N, K) * M * N, device=DEV)
        ops.gemm_mid(None, x, w, mode=2, partial=part)
        outs.append(part)
        if N % 32 == 0:
            out = torch.empty(M, N // 2, dtype=torch.bfloat16, device=DEV)
            ops.gemm_mid(out, x, w, bias, mode=1)
            outs.append(out)
        results.append(outs)
    for a, b in zip(*results):
        bits = torch.int16 if a.dtype == torch.bfloat16 else torch.int32
        assert torch.equal(a.view(bits), b.view(bits))
    assert torch.allclose(results[0][1], x.float() @ w.float().t() + bias.float(), atol=3e-2, rtol=2e-2)


def test_linear_picks_a_kernel_by_row_count(ops):
    w = rnd(96, 256, dtype=torch.bfloat16, seed=5, scale=0.05)
    for M in (3, 64, 65, 200):
        x = rnd(M, 256, dtype=torch.bfloat16, seed=M)
        out = torch.empty(M, 96, dtype=torch.bfloat16, device=DEV)
        ops.linear(out, x, w)
        assert torch.allclose(out.double(), x.double() @ w.double().T, atol=2e-2, rtol=2e-2)
    # a float32 result keeps the float32 sums unrounded on every path (few rows: our kernel;
    # more: the vendor product asked for float32)
    bias = rnd(96, dtype=torch.bfloat16, seed=9)
    for M in (3, 12, 40, 100, 200):
        x = rnd(M, 256, dtype=torch.bfloat16, seed=M)
        for b in (None, bias):
            out = torch.empty(M, 96, device=DEV)
            ops.linear(out, x, w, b)
            want = x.double() @ w.double().T + (0 if b is None else b.double())
            assert torch.allclose(out.double(), want, atol=2e-6, rtol=2e-6), (M, b is not None)


@pytest.mark.parametrize("M", [5, 12, 40, 100])
def test_bf16_products_sum_in_float32(ops, M):
    """Inputs of one sign and a long K: every product is 1 + 2^-7 exactly and every partial sum
    is a multiple of 2^-7 below 2^24, so float32 sums are exact in any order (4128), while a
    sum kept in bfloat16 would stall at 256."""
    K, N = 4096, 128
    x = torch.ones(M, K, dtype=torch.bfloat16, device=DEV)
    w = torch.full((N, K), 1.0 + 2.0 ** -7, dtype=torch.bfloat16, device=DEV)
    want = torch.full((M, N), 4096 * (1.0 + 2.0 ** -7), device=DEV)
    out = torch.empty(M, N, device=DEV)
    ops.linear(out, x, w)
    assert torch.equal(out, want)
    out16 = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    ops.linear(out16, x, w)
    assert torch.equal(out16.float(), want.to(torch.bfloat16).float())  # rounded once, at the end
    if M <= ops.SKINNY_MAX_ROWS:
        out.zero_()
        ops.gemm_skinny_bf16(out, x, w)
        assert torch.equal(out, want)
        out.zero_()
        ops.gemm_mid(out, x, w, mode=0)
        assert torch.equal(out, want)


def test_logits_finish_bias_cap_and_scale(ops):
    """kvcore/sample/logits_processor.py:44-54: bias, then the soft cap, then the scale; the
    reference's own vector (tests/test_sampler.py:20-26): logits [2, -2] under a cap of 1
    stay within [-1, 1]."""
    logits = torch.tensor([[2.0, -2.0]], device=DEV)
    ops.logits_finish(logits, None, 1.0, 1.0)
    assert torch.allclose(logits.cpu(), torch.tanh(torch.tensor([[2.0, -2.0]])), atol=1e-6)
    assert (logits.abs() <= 1.0).all()
    x = rnd(7, 1001, seed=3, scale=3.0)
    wide = torch.zeros(7, 1100, device=DEV)
    wide[:, :1001] = x
    for bias in (None, rnd(1001, dtype=torch.bfloat16, seed=4), rnd(1001, seed=5)):
        got = wide.clone()
        ops.logits_finish(got[:, :1001], bias, 2.5, 0.5)
        want = x.double() + (0 if bias is None else bias.double())
        want = torch.tanh(want / 2.5) * 2.5 * 0.5
        assert torch.allclose(got[:, :1001].double(), want, atol=1e-6)
        assert (got[:, 1001:] == 0).all()
    plainly = x.clone()
    ops.logits_finish(plainly, None, 0.0, 1.0)
    assert torch.equal(plainly, x)


def test_fill_pages_touches_the_listed_pages_only(ops):
    for dtype in DTYPES:
        kv = torch.zeros(3, 2, 9, 2, 4, 16, dtype=dtype, device=DEV)  # [planes, k/v, pages, heads, page, d]
        triples = torch.tensor([0, 0, 4, 1, 1, 0, 0, 1, 7, 2, 0, 99], dtype=torch.int32, device=DEV)
        ops.fill_pages(kv, triples[2:], 4, float("nan"), stride=3)  # pages 4, 0 (null), 7, 99 (outside)
        nan_pages = torch.isnan(kv.float()).flatten(3).all(dim=3)     # [3, 2, 9]
        any_nan = torch.isnan(kv.float()).flatten(3).any(dim=3)
        assert nan_pages[:, :, [4, 7]].all()
        assert not any_nan[:, :, [0, 1, 2, 3, 5, 6, 8]].any()
        pages = torch.tensor([1, 8], dtype=torch.int32, device=DEV)
        ops.fill_pages(kv, pages, 2, 0.5)
        assert (kv[:, :, [1, 8]] == 0.5).all() and (kv[:, :, 2] == 0).all()


def test_random_fill_gives_the_host_generator_bits(ops):
    """The kernel and its host twin draw the same values for one seed, in float32 and rounded
    to bfloat16, so a model drawn on the GPU is the model that a written folder holds."""
    import numpy as np

    from kvcore_amd.weights import random_normal

    n = 3_000_017  # covers every table entry and both tails many times over
    for lo, hi, mean, std in ((123, 456, 0.0, 0.02), (0xFFFFFFFF, 7, 1.0, 0.1)):
        want = torch.from_numpy(random_normal.normal(lo, hi, n, mean, std))
        got = torch.empty(n, device=DEV)
        ops.fill_normal(got, lo, hi, mean, std)
        assert torch.equal(got.cpu().view(torch.int32), want.view(torch.int32))
        got16 = torch.empty(n, dtype=torch.bfloat16, device=DEV)
        ops.fill_normal(got16, lo, hi, mean, std)
        assert torch.equal(got16.cpu().view(torch.int16), want.to(torch.bfloat16).view(torch.int16))
    z = (want.double() - 1.0) / 0.1
    assert abs(float(z.mean())) < 3e-3 and abs(float(z.std()) - 1.0) < 3e-3
    assert 4.5 < float(z.abs().max()) < 6.5
    # an index beyond 32 bits changes the draw (the high word is mixed in)
    a = random_normal.standard_normal(1, 2, 5, 4)
    b = random_normal.standard_normal(1, 2, 5 + (1 << 32), 4)
    assert not np.array_equal(a, b)


def test_rope_table(ops):
    pos = torch.tensor([0, 1, 77, 4095, 100000], dtype=torch.int32, device=DEV)
    inv = plain.rope_inv_freq(48, 25000.0).float().to(DEV)
    cos = torch.empty(5, 24, device=DEV)
    sin = torch.empty(5, 24, device=DEV)
    ops.rope_table(cos, sin, pos, inv)
    ang = (pos.float()[:, None] * inv[None, :]).double()  # the angle itself is float32
    assert torch.allclose(cos.double(), ang.cos(), atol=2e-7)
    assert torch.allclose(sin.double(), ang.sin(), atol=2e-7)


def make_cache(pages, nkv, page_size, d, dtype):
    """K pages [pages, nkv, page_size, d]; V pages [pages, nkv, d, page_size]; all NaN."""
    k = torch.full((pages, nkv, page_size, d), float("nan"), dtype=dtype, device=DEV)
    return k, k.clone().view(pages, nkv, d, page_size)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("interleaved,rot_dim", [(False, 32), (True, 32), (False, 16), (False, 8), (False, 0)])
def test_rope_kv_write(ops, dtype, interleaved, rot_dim):
    nh, nkv, d, page = 3, 1, 32, 4
    T = 6
    qkv0 = rnd(T, (nh + 2 * nkv) * d, dtype=dtype)
    positions = torch.tensor([5, 6, 7, 0, 1, 9], dtype=torch.int32, device=DEV)
    token_req = torch.tensor([0, 0, 0, 1, 1, -1], dtype=torch.int32, device=DEV)
    slots = torch.tensor([2, 0], dtype=torch.int32, device=DEV)
    table = torch.zeros(3, 4, dtype=torch.int32, device=DEV)
    table[2, :2] = torch.tensor([5, 3])
    table[0, :1] = torch.tensor([1])
    kc, vc = make_cache(7, nkv, page, d, dtype)
    half = rot_dim // 2
    inv = plain.rope_inv_freq(rot_dim, 10000.0).float().to(DEV) if rot_dim else torch.zeros(0, device=DEV)
    cos = torch.empty(T, half, device=DEV)
    sin = torch.empty(T, half, device=DEV)
    if rot_dim:
        ops.rope_table(cos, sin, positions, inv)
    qkv = qkv0.clone()
    kv_slot = torch.empty(T, dtype=torch.int32, device=DEV)
    ops.kv_slots(kv_slot, positions=positions, token_req=token_req, slots=slots, table=table,
                 page_size=page, num_pages=7)
    assert kv_slot.cpu().tolist() == [3 * 4 + 1, 3 * 4 + 2, 3 * 4 + 3, 1 * 4 + 0, 1 * 4 + 1, -2]
    ops.rope_kv_write(qkv, kc, vc, cos, sin, rot_dim=rot_dim, interleaved=interleaved,
                      kv_slot=kv_slot, nh=nh, nkv=nkv, d=d)

    def rotate(x):  # x [T, heads, d] float64
        if not rot_dim:
            return x
        part = x[..., :rot_dim]
        if interleaved:
            part = torch.cat((part[..., 0::2], part[..., 1::2]), dim=-1)
        y = plain.apply_rope(part, positions.cpu().long(), inv.double().cpu())
        if interleaved:
            z = torch.empty_like(y)
            z[..., 0::2], z[..., 1::2] = y[..., :half], y[..., half:]
            y = z
        return torch.cat((y, x[..., rot_dim:]), dim=-1)

    x = qkv0.double().cpu().view(T, nh + 2 * nkv, d)
    want_q = rotate(x[:, :nh])
    want_k = rotate(x[:, nh:nh + nkv])
    got = qkv.double().cpu().view(T, nh + 2 * nkv, d)
    live = [0, 1, 2, 3, 4]
    assert torch.allclose(got[live, :nh], want_q[live], **tol(dtype))
    assert torch.equal(got[5], x[5])  # a padding token is left alone
    assert torch.equal(got[:, nh + nkv:], x[:, nh + nkv:])  # v is never rotated
    where = {0: (3, 1), 1: (3, 2), 2: (3, 3), 3: (1, 0), 4: (1, 1)}  # token -> (page, offset)
    for t, (pg, off) in where.items():
        assert torch.allclose(kc[pg, 0, off].double().cpu(), want_k[t, 0], **tol(dtype))
        assert torch.equal(vc[pg, 0, :, off].double().cpu(), x[t, nh + nkv])
    written = torch.zeros(7, page, dtype=torch.bool)
    for pg, off in where.values():
        written[pg, off] = True
    assert torch.isnan(kc[:, 0, :, 0].cpu()[~written]).all()  # nothing else was touched
    # write_kv off: q is rotated, the cache is not written
    kc2, vc2 = make_cache(7, nkv, page, d, dtype)
    qkv = qkv0.clone()
    ops.rope_kv_write(qkv, kc2, vc2, cos, sin, rot_dim=rot_dim, interleaved=interleaved,
                      kv_slot=kv_slot, nh=nh, nkv=nkv, d=d, write_kv=False)
    assert torch.isnan(kc2).all() and torch.isnan(vc2).all()
    assert torch.allclose(qkv.double().cpu().view(T, -1, d)[live, :nh], want_q[live], **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,d,rot_dim,page", [(4, 2, 64, 64, 16), (3, 1, 32, 16, 8), (2, 2, 128, 64, 48)])
@pytest.mark.parametrize("rotate_q", [True, False])
def test_rope_kv_write_of_many_tokens_equals_token_by_token(ops, dtype, nh, nkv, d, rot_dim, page, rotate_q):
    """Steps of 16 tokens and more take a kernel that handles eight tokens a block and stores
    the values of eight neighbours in a page together.  It must leave the bits that the kernel
    for few tokens leaves: requests that start in mid-page, a run that crosses a page, a
    padding token, a token without a page, a ragged last block."""
    lens = [(5, 37), (0, 9), (24, 30)]  # (first position, tokens) per request
    positions, token_req = [], []
    for r, (first, n) in enumerate(lens):
        positions += list(range(first, first + n))
        token_req += [r] * n
    positions += [0, 20]
    token_req += [-1, 1]  # a padding token, and one more token of request 1, apart from its others
    T = len(positions)
    positions = torch.tensor(positions, dtype=torch.int32, device=DEV)
    token_req = torch.tensor(token_req, dtype=torch.int32, device=DEV)
    slots = torch.tensor([2, 0, 1], dtype=torch.int32, device=DEV)
    pages_per = -(-60 // page)
    n_pages = 3 * pages_per + 1
    table = torch.zeros(3, pages_per + 1, dtype=torch.int32, device=DEV)
    order = torch.randperm(n_pages - 1, generator=torch.Generator().manual_seed(3)) + 1
    for row in range(3):
        table[row, :pages_per] = order[row * pages_per:(row + 1) * pages_per].to(torch.int32)
    table[1, 53 // page] = 0  # request 2 (slot 1) has no page for its last positions: they are not stored
    kv_slot = torch.empty(T, dtype=torch.int32, device=DEV)
    ops.kv_slots(kv_slot, positions=positions, token_req=token_req, slots=slots, table=table,
                 page_size=page, num_pages=n_pages)
    assert (kv_slot == -1).any() and (kv_slot == -2).any()
    inv = plain.rope_inv_freq(rot_dim, 10000.0).float().to(DEV)
    cos = torch.empty(T, rot_dim // 2, device=DEV)
    sin = torch.empty(T, rot_dim // 2, device=DEV)
    ops.rope_table(cos, sin, positions, inv)
    qkv0 = rnd(T, (nh + 2 * nkv) * d, dtype=dtype, seed=4)
    results = []
    for step in (T, 7):  # all at once, then seven tokens a call
        qkv = qkv0.clone()
        kc, vc = make_cache(n_pages, nkv, page, d, dtype)
        for a in range(0, T, step):
            b = min(a + step, T)
            ops.rope_kv_write(qkv[a:b], kc, vc, cos[a:b], sin[a:b], rot_dim=rot_dim, interleaved=False,
                              kv_slot=kv_slot[a:b], nh=nh, nkv=nkv, d=d, rotate_q=rotate_q)
        results.append((qkv, kc, vc))
    bits = torch.int16 if dtype == torch.bfloat16 else torch.int32
    for one, other in zip(results[0], results[1]):
        assert torch.equal(one.view(bits), other.view(bits))
    assert not torch.isnan(results[0][1]).all() and torch.isnan(results[0][1]).any()


def test_kv_slots_vector_of_the_reference(ops):
    """tests/test_block_table.py:65-85: rows [3,4] and [5], page size 2, positions
    [0,1,2,3,0,1] -> slots [6,7,8,9,10,11]; beyond the row's pages there is no slot."""
    table = torch.zeros(2, 3, dtype=torch.int32, device=DEV)
    table[0, :2] = torch.tensor([3, 4], dtype=torch.int32)
    table[1, :1] = torch.tensor([5], dtype=torch.int32)
    positions = torch.tensor([0, 1, 2, 3, 0, 1, 2, 0], dtype=torch.int32, device=DEV)
    token_req = torch.tensor([0, 0, 0, 0, 1, 1, 1, -1], dtype=torch.int32, device=DEV)
    out = torch.empty(8, dtype=torch.int32, device=DEV)
    ops.kv_slots(out, positions=positions, token_req=token_req,
                 slots=torch.tensor([0, 1], dtype=torch.int32, device=DEV), table=table,
                 page_size=2, num_pages=8)
    assert out.cpu().tolist() == [6, 7, 8, 9, 10, 11, -1, -2]


def paged_setup(seq_lens, nkv, d, page, dtype, seed=0, shuffle=True):
    """Random K/V for requests of the given lengths, scattered over shuffled pages of a
    NaN-filled cache.  Returns cache planes, table, and the dense K/V per request."""
    g = torch.Generator().manual_seed(seed)
    n_pages = sum(-(-n // page) for n in seq_lens) + 3
    order = torch.randperm(n_pages - 1, generator=g) + 1 if shuffle else torch.arange(1, n_pages)
    kc, vc = make_cache(n_pages, nkv, page, d, dtype)
    table = torch.zeros(len(seq_lens) + 2, max(-(-n // page) for n in seq_lens) + 1, dtype=torch.int32)
    dense = []
    at = 0
    for r, n in enumerate(seq_lens):
        k = (torch.randn(n, nkv, d, generator=g)).to(dtype)
        v = (torch.randn(n, nkv, d, generator=g)).to(dtype)
        dense.append((k, v))
        for i in range(-(-n // page)):
            pg = int(order[at]); at += 1
            table[r + 1, i] = pg  # request r lives in slot r + 1
            lo, hi = i * page, min((i + 1) * page, n)
            kc[pg, :, : hi - lo] = k[lo:hi].transpose(0, 1).to(DEV)
            vc[pg, :, :, : hi - lo] = v[lo:hi].permute(1, 2, 0).to(DEV)
    return kc, vc, table.to(DEV), dense


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,d,page", [(4, 2, 16, 4), (3, 1, 48, 16), (8, 8, 128, 32), (2, 1, 256, 8)])
def test_paged_attention_mixed_batch(ops, dtype, nh, nkv, d, page):
    seq_lens = [70, 1, 33, 130]
    q_lens = [70, 1, 5, 1]  # a whole prompt, a first token, a portion with context, a decode
    kc, vc, table, dense = paged_setup(seq_lens, nkv, d, page, dtype, seed=d)
    T = sum(q_lens)
    q = rnd(T, nh * d, dtype=dtype, seed=7)
    positions, token_req = [], []
    for r, (n, ql) in enumerate(zip(seq_lens, q_lens)):
        positions += list(range(n - ql, n))
        token_req += [r] * ql
    positions = torch.tensor(positions, dtype=torch.int32, device=DEV)
    token_req_t = torch.tensor(token_req, dtype=torch.int32, device=DEV)
    slots = torch.tensor([1, 2, 3, 4], dtype=torch.int32, device=DEV)
    out = torch.empty(T, nh * d, dtype=dtype, device=DEV)
    scale = d ** -0.5
    ops.paged_attention(out, q, kc, vc, table=table, positions=positions, token_req=token_req_t,
                        slots=slots, nh=nh, nkv=nkv, d=d, scale=scale)
    got = out.double().cpu().view(T, nh, d)
    qd = q.double().cpu().view(T, nh, d)
    t = 0
    for r, (n, ql) in enumerate(zip(seq_lens, q_lens)):
        k, v = dense[r][0].double(), dense[r][1].double()
        full_q = torch.zeros(n, nh, d, dtype=torch.float64)
        full_q[n - ql:] = qd[t:t + ql]
        want = plain.causal_gqa_attention(full_q, k, v, scale)[n - ql:]
        assert torch.allclose(got[t:t + ql], want, **tol(dtype)), f"request {r}"
        t += ql


@pytest.mark.parametrize("dtype", DTYPES)
def test_paged_attention_finds_one_far_key_among_hundreds(ops, dtype):
    """Random keys would hide a skipped key.  One key (in turn: the first, one at a page's
    edge, the last of a page, the query's own) is made to match the query with a large
    score; the output must be that key's value."""
    nh, nkv, d, page = 2, 1, 64, 16
    n = 700
    for special in [0, 15, 16, 351, 639, 640, 698, 699]:
        kc, vc, table, dense = paged_setup([n], nkv, d, page, dtype, seed=special)
        q = rnd(1, nh * d, dtype=dtype, seed=3)
        qd = q.float().view(nh, d)
        key = (qd[0] + qd[1]) / 2  # matches both heads
        key = key * (60.0 / float((qd[0] * key).sum() * d ** -0.5))  # score about 60 after scaling
        pg, off = int(table[1, special // page]), special % page
        kc[pg, 0, off] = key.to(dtype)
        positions = torch.tensor([n - 1], dtype=torch.int32, device=DEV)
        out = torch.empty(1, nh * d, dtype=dtype, device=DEV)
        ops.paged_attention(out, q, kc, vc, table=table, positions=positions,
                            token_req=torch.zeros(1, dtype=torch.int32, device=DEV),
                            slots=torch.ones(1, dtype=torch.int32, device=DEV),
                            nh=nh, nkv=nkv, d=d, scale=d ** -0.5)
        want = vc[pg, 0, :, off].double().cpu()
        got = out.double().cpu().view(nh, d)[0]
        assert torch.allclose(got, want, atol=2e-2 if dtype == torch.bfloat16 else 1e-4), special


@pytest.mark.parametrize("dtype", DTYPES)
def test_paged_attention_window_edge(ops, dtype):
    nh, nkv, d, page, n, w = 2, 2, 32, 8, 90, 20
    kc, vc, table, dense = paged_setup([n], nkv, d, page, dtype, seed=11)
    q_len = 30
    q = rnd(q_len, nh * d, dtype=dtype, seed=5)
    positions = torch.arange(n - q_len, n, dtype=torch.int32, device=DEV)
    out = torch.empty(q_len, nh * d, dtype=dtype, device=DEV)
    args = dict(table=table, positions=positions, token_req=torch.zeros(q_len, dtype=torch.int32, device=DEV),
                slots=torch.ones(1, dtype=torch.int32, device=DEV), nh=nh, nkv=nkv, d=d, scale=0.2)
    ops.paged_attention(out, q, kc, vc, window=w, **args)
    k, v = dense[0][0].double(), dense[0][1].double()
    full_q = torch.zeros(n, nh, d, dtype=torch.float64)
    full_q[n - q_len:] = q.double().cpu().view(q_len, nh, d)
    want = plain.causal_gqa_attention(full_q, k, v, 0.2, window=w)[n - q_len:]
    assert torch.allclose(out.double().cpu().view(q_len, nh, d), want, **tol(dtype))
    # pages wholly behind the window may be gone (null page): the result does not change
    first_needed = (n - q_len) - w + 1
    table2 = table.clone()
    table2[1, : first_needed // page] = 0
    out2 = torch.empty_like(out)
    ops.paged_attention(out2, q, kc, vc, window=w, **{**args, "table": table2})
    assert torch.equal(out, out2)
    # the key at the window's edge counts, the one before it does not
    edge = n - 1 - w + 1
    big = torch.zeros(d)
    big[0] = 1.0
    qq = torch.zeros(1, nh * d, dtype=dtype, device=DEV)
    qq[0, 0] = 300.0
    qq[0, d] = 300.0
    for pos_key, seen in ((edge, True), (edge - 1, False)):
        kc2 = kc.clone()
        kc2[:, :, :, 0] = 0
        pg, off = int(table[1, pos_key // page]), pos_key % page
        kc2[pg, :, off, 0] = 1.0
        o = torch.empty(1, nh * d, dtype=dtype, device=DEV)
        ops.paged_attention(o, qq, kc2, vc, window=w, **{**args, "positions": positions[-1:],
                                                         "token_req": torch.zeros(1, dtype=torch.int32, device=DEV)})
        hit = torch.allclose(o.float().cpu().view(nh, d), vc[pg, :, :, off].float().cpu(), atol=2e-2)
        assert hit == seen


@pytest.mark.parametrize("nh,nkv,d,page", [(4, 1, 32, 16), (6, 2, 64, 16), (32, 8, 128, 16), (16, 1, 128, 32),
                                           (3, 3, 96, 48), (8, 2, 256, 16)])
@pytest.mark.parametrize("nsplit", [1, 3, 16])
def test_decode_attention_on_the_matrix_cores(ops, nh, nkv, d, page, nsplit):
    """Single tokens of several requests at once, against the plain attention, with the
    key range cut into parts; lengths chosen at block and page edges."""
    dtype = torch.bfloat16
    assert ops.decode_attention_supported(nh, nkv, d, page, dtype)
    seq_lens = [1, 15, 16, 17, 95, 96, 97, 300, 641]
    R = len(seq_lens)
    kc, vc, table, dense = paged_setup(seq_lens, nkv, d, page, dtype, seed=d + nsplit)
    q = rnd(R + 1, nh * d, dtype=dtype, seed=2)  # one padding token at the end
    positions = torch.tensor([n - 1 for n in seq_lens] + [0], dtype=torch.int32, device=DEV)
    token_req = torch.tensor(list(range(R)) + [-1], dtype=torch.int32, device=DEV)
    slots = torch.arange(1, R + 1, dtype=torch.int32, device=DEV)
    out = torch.full((R + 1, nh * d), float("nan"), dtype=dtype, device=DEV)
    part_o = torch.full(((R + 1) * nh * nsplit, d), float("nan"), device=DEV)
    part_ml = torch.full(((R + 1) * nh * nsplit, 2), float("nan"), device=DEV)
    scale = d ** -0.5
    ops.decode_attention(out, q, kc, vc, table=table, positions=positions, token_req=token_req,
                         slots=slots, nh=nh, nkv=nkv, d=d, scale=scale, nsplit=nsplit,
                         part_o=part_o, part_ml=part_ml)
    got = out.double().cpu().view(R + 1, nh, d)
    assert torch.all(got[R] == 0)
    qd = q.double().cpu().view(R + 1, nh, d)
    for r, n in enumerate(seq_lens):
        k, v = dense[r][0].double(), dense[r][1].double()
        full_q = torch.zeros(n, nh, d, dtype=torch.float64)
        full_q[n - 1] = qd[r]
        want = plain.causal_gqa_attention(full_q, k, v, scale)[n - 1]
        assert torch.allclose(got[r], want, atol=1e-2, rtol=1e-2), f"length {n}"
    # the general kernel gives the same answer
    ref = torch.empty_like(out)
    ops.paged_attention(ref, q, kc, vc, table=table, positions=positions, token_req=token_req,
                        slots=slots, nh=nh, nkv=nkv, d=d, scale=scale)
    assert torch.allclose(out.float(), ref.float(), atol=1e-2, rtol=1e-2)


@pytest.mark.parametrize("nh,nkv,d,page", [(4, 1, 32, 16), (32, 8, 128, 16), (6, 2, 64, 32), (8, 2, 256, 16),
                                           (3, 3, 96, 48), (16, 1, 160, 16)])
@pytest.mark.parametrize("rot,interleaved", [("full", False), ("half", False), ("full", True), ("none", False)])
@pytest.mark.parametrize("nsplit", [1, 3])
def test_decode_attention_rotates_and_writes_like_the_separate_kernels(ops, nh, nkv, d, page, rot,
                                                                        interleaved, nsplit):
    """The decode kernel with rotation and cache write built in gives the bits of
    rope_kv_write followed by the attention alone: outputs, and every byte of the cache."""
    dtype = torch.bfloat16
    seq_lens = [1, 15, 16, 17, 96, 97, 300, 641]
    R = len(seq_lens)
    kc, vc, table, dense = paged_setup(seq_lens, nkv, d, page, dtype, seed=d + nsplit)
    for r, n in enumerate(seq_lens):  # the token's own slot is not written yet
        pg, off = int(table[r + 1, (n - 1) // page]), (n - 1) % page
        kc[pg, :, off] = float("nan")
        vc[pg, :, :, off] = float("nan")
    T = R + 1  # one padding token at the end
    qkv0 = rnd(T, (nh + 2 * nkv) * d, dtype=dtype, seed=9)
    positions = torch.tensor([n - 1 for n in seq_lens] + [0], dtype=torch.int32, device=DEV)
    token_req = torch.tensor(list(range(R)) + [-1], dtype=torch.int32, device=DEV)
    slots = torch.arange(1, R + 1, dtype=torch.int32, device=DEV)
    rot_dim = {"full": d, "half": d // 2, "none": 0}[rot]
    cos = torch.empty(T, rot_dim // 2, device=DEV)
    sin = torch.empty(T, rot_dim // 2, device=DEV)
    if rot_dim:
        inv = plain.rope_inv_freq(rot_dim, 10000.0).float().to(DEV)
        ops.rope_table(cos, sin, positions, inv)
    part_o = torch.full((T * nh * nsplit, d), float("nan"), device=DEV)
    part_ml = torch.full((T * nh * nsplit, 2), float("nan"), device=DEV)
    common = dict(table=table, positions=positions, token_req=token_req, slots=slots, nh=nh, nkv=nkv,
                  d=d, scale=d ** -0.5, nsplit=nsplit, part_o=part_o, part_ml=part_ml)

    kc1, vc1, qkv1 = kc.clone(), vc.clone(), qkv0.clone()
    kv_slot = torch.empty(T, dtype=torch.int32, device=DEV)
    ops.kv_slots(kv_slot, positions=positions, token_req=token_req, slots=slots, table=table,
                 page_size=page, num_pages=kc.shape[0])
    ops.rope_kv_write(qkv1, kc1, vc1, cos, sin, rot_dim=rot_dim, interleaved=interleaved,
                      kv_slot=kv_slot, nh=nh, nkv=nkv, d=d)
    out1 = torch.full((T, nh * d), float("nan"), dtype=dtype, device=DEV)
    ops.decode_attention(out1, qkv1, kc1, vc1, **common)
    assert not torch.isnan(out1).any()

    kc2, vc2, qkv2 = kc.clone(), vc.clone(), qkv0.clone()
    out2 = torch.full((T, nh * d), float("nan"), dtype=dtype, device=DEV)
    token_rows = torch.tensor(list(range(1, R + 1)) + [-1], dtype=torch.int32, device=DEV)
    ops.decode_attention(out2, qkv2, kc2, vc2, cos=cos, sin=sin, rot_dim=rot_dim,
                         interleaved=interleaved, write_kv=True,
                         token_rows=token_rows if nsplit == 1 else None, **common)
    bits = lambda x: x.view(torch.int16)
    assert torch.equal(bits(qkv2), bits(qkv0))
    assert torch.equal(bits(out2), bits(out1))
    assert torch.equal(bits(kc2), bits(kc1)) and torch.equal(bits(vc2), bits(vc1))

    # without the write the cache must already hold the token (a layer that reads another's cache)
    out3 = torch.full((T, nh * d), float("nan"), dtype=dtype, device=DEV)
    kc3, vc3 = kc1.clone(), vc1.clone()
    ops.decode_attention(out3, qkv0, kc3, vc3, cos=cos, sin=sin, rot_dim=rot_dim,
                         interleaved=interleaved, write_kv=False, **common)
    assert torch.equal(bits(out3), bits(out1))
    assert torch.equal(bits(kc3), bits(kc1)) and torch.equal(bits(vc3), bits(vc1))


@pytest.mark.parametrize("nsplit", [1, 5])
def test_decode_attention_far_key_and_window(ops, nsplit):
    dtype = torch.bfloat16
    nh, nkv, d, page, n = 8, 2, 64, 16, 700
    part_o = torch.empty(nh * nsplit, d, device=DEV)
    part_ml = torch.empty(nh * nsplit, 2, device=DEV)
    args = dict(positions=torch.tensor([n - 1], dtype=torch.int32, device=DEV),
                token_req=torch.zeros(1, dtype=torch.int32, device=DEV),
                slots=torch.ones(1, dtype=torch.int32, device=DEV), nh=nh, nkv=nkv, d=d,
                scale=d ** -0.5, nsplit=nsplit, part_o=part_o, part_ml=part_ml)
    for special in [0, 15, 16, 351, 639, 640, 698, 699]:
        kc, vc, table, dense = paged_setup([n], nkv, d, page, dtype, seed=special)
        q = rnd(1, nh * d, dtype=dtype, seed=3)
        qd = q.float().view(nh, d)
        key = qd[:4].mean(0)  # matches the four heads of kv head 0
        key = key * (60.0 / float((qd[0] * key).sum() * d ** -0.5))
        pg, off = int(table[1, special // page]), special % page
        kc[pg, 0, off] = key.to(dtype)
        out = torch.empty(1, nh * d, dtype=dtype, device=DEV)
        ops.decode_attention(out, q, kc, vc, table=table, **args)
        assert torch.allclose(out.float().cpu().view(nh, d)[0], vc[pg, 0, :, off].float().cpu(), atol=3e-2), special
    # window: only the last w keys count; pages behind it may be the null page
    w = 40
    kc, vc, table, dense = paged_setup([n], nkv, d, page, dtype, seed=77)
    q = rnd(1, nh * d, dtype=dtype, seed=4)
    out = torch.empty(1, nh * d, dtype=dtype, device=DEV)
    table2 = table.clone()
    table2[1, : (n - w) // page] = 0
    ops.decode_attention(out, q, kc, vc, table=table2, window=w, **args)
    k, v = dense[0][0].double(), dense[0][1].double()
    full_q = torch.zeros(n, nh, d, dtype=torch.float64)
    full_q[n - 1] = q.double().cpu().view(nh, d)
    want = plain.causal_gqa_attention(full_q, k, v, d ** -0.5, window=w)[n - 1]
    assert torch.allclose(out.double().cpu().view(nh, d), want, atol=1e-2, rtol=1e-2)


@pytest.mark.parametrize("nh,nkv,d,page", [(8, 2, 64, 16), (32, 8, 128, 16), (6, 2, 128, 32), (5, 1, 64, 48),
                                           (4, 4, 128, 16), (16, 1, 64, 16)])
@pytest.mark.parametrize("nsplit", [1, 3])
def test_prefill_attention_on_the_matrix_cores(ops, nh, nkv, d, page, nsplit):
    """Portions of prompts with and without earlier context, beside single tokens, against
    the plain attention; lengths chosen at tile, block and page edges.  With the keys of a
    tile dealt to three blocks, the short requests leave some of the three without keys."""
    dtype = torch.bfloat16
    assert ops.prefill_attention_supported(nh, nkv, d, page, dtype)
    seq_lens = [200, 1, 33, 130, 64, 97, 700]
    q_lens = [200, 1, 5, 1, 64, 17, 129]
    kc, vc, table, dense = paged_setup(seq_lens, nkv, d, page, dtype, seed=d + nh)
    T = sum(q_lens)
    q = rnd(T, nh * d, dtype=dtype, seed=7)
    positions, q_start = [], [0]
    for n, ql in zip(seq_lens, q_lens):
        positions += list(range(n - ql, n))
        q_start.append(q_start[-1] + ql)
    positions = torch.tensor(positions, dtype=torch.int32, device=DEV)
    q_start_t = torch.tensor(q_start, dtype=torch.int32, device=DEV)
    slots = torch.arange(1, len(seq_lens) + 1, dtype=torch.int32, device=DEV)
    out = torch.full((T, nh * d), float("nan"), dtype=dtype, device=DEV)
    scale = d ** -0.5
    part_o = torch.full((T * nh * nsplit, d), float("nan"), device=DEV)
    part_ml = torch.full((T * nh * nsplit, 2), float("nan"), device=DEV)
    ops.prefill_attention(out, q, kc, vc, table=table, positions=positions, q_start=q_start_t,
                          slots=slots, num_reqs=len(seq_lens), nh=nh, nkv=nkv, d=d, scale=scale,
                          nsplit=nsplit, part_o=part_o, part_ml=part_ml)
    got = out.double().cpu().view(T, nh, d)
    qd = q.double().cpu().view(T, nh, d)
    for r, (n, ql) in enumerate(zip(seq_lens, q_lens)):
        k, v = dense[r][0].double(), dense[r][1].double()
        full_q = torch.zeros(n, nh, d, dtype=torch.float64)
        full_q[n - ql:] = qd[q_start[r]:q_start[r + 1]]
        want = plain.causal_gqa_attention(full_q, k, v, scale)[n - ql:]
        assert torch.allclose(got[q_start[r]:q_start[r + 1]], want, atol=1e-2, rtol=1e-2), f"request {r}"


@pytest.mark.parametrize("nsplit", [1, 4])
def test_prefill_attention_far_key_and_window(ops, nsplit):
    dtype = torch.bfloat16
    nh, nkv, d, page, n, ql = 8, 2, 64, 16, 700, 40
    positions = torch.arange(n - ql, n, dtype=torch.int32, device=DEV)
    args = dict(positions=positions, q_start=torch.tensor([0, ql], dtype=torch.int32, device=DEV),
                slots=torch.ones(1, dtype=torch.int32, device=DEV), num_reqs=1, nh=nh, nkv=nkv, d=d,
                scale=d ** -0.5, nsplit=nsplit, part_o=torch.empty(ql * nh * nsplit, d, device=DEV),
                part_ml=torch.empty(ql * nh * nsplit, 2, device=DEV))
    for special in [0, 15, 16, 63, 64, 351, 659, 660, 698, 699]:
        kc, vc, table, dense = paged_setup([n], nkv, d, page, dtype, seed=special)
        q = rnd(ql, nh * d, dtype=dtype, seed=3)
        qd = q.float().view(ql, nh, d)
        key = qd[-1, :4].mean(0)  # matches the last token's heads of kv head 0
        key = key * (60.0 / float((qd[-1, 0] * key).sum() * d ** -0.5))
        pg, off = int(table[1, special // page]), special % page
        kc[pg, 0, off] = key.to(dtype)
        out = torch.empty(ql, nh * d, dtype=dtype, device=DEV)
        ops.prefill_attention(out, q, kc, vc, table=table, **args)
        assert torch.allclose(out.float().cpu().view(ql, nh, d)[-1, 0], vc[pg, 0, :, off].float().cpu(),
                              atol=3e-2), special
    w = 50
    kc, vc, table, dense = paged_setup([n], nkv, d, page, dtype, seed=78)
    q = rnd(ql, nh * d, dtype=dtype, seed=4)
    table2 = table.clone()
    table2[1, : (n - ql - w + 1) // page] = 0  # pages wholly behind the first row's window are gone
    out = torch.empty(ql, nh * d, dtype=dtype, device=DEV)
    ops.prefill_attention(out, q, kc, vc, table=table2, window=w, **args)
    k, v = dense[0][0].double(), dense[0][1].double()
    full_q = torch.zeros(n, nh, d, dtype=torch.float64)
    full_q[n - ql:] = q.double().cpu().view(ql, nh, d)
    want = plain.causal_gqa_attention(full_q, k, v, d ** -0.5, window=w)[n - ql:]
    assert torch.allclose(out.double().cpu().view(ql, nh, d), want, atol=1e-2, rtol=1e-2)


@pytest.mark.parametrize("nh,nkv,d,rot_dim,interleaved", [(8, 2, 128, 128, False), (8, 2, 128, 64, False),
                                                          (6, 3, 64, 64, False), (4, 1, 128, 96, True),
                                                          (4, 4, 64, 32, True)])
@pytest.mark.parametrize("nsplit", [1, 3])
def test_prefill_attention_rotates_the_queries_like_the_separate_kernel(ops, nh, nkv, d, rot_dim, interleaved,
                                                                        nsplit):
    """Unrotated queries with the rotary tables give, bit for bit, what the rotation in memory
    followed by the kernel without tables gives; the rotation without ``rotate_q`` leaves the
    query heads alone and still rotates and stores the keys."""
    dtype, page = torch.bfloat16, 16
    seq_lens, q_lens = [300, 77], [130, 77]
    kc, vc, table, _ = paged_setup(seq_lens, nkv, d, page, dtype, seed=11)
    T = sum(q_lens)
    qkv0 = rnd(T, (nh + 2 * nkv) * d, dtype=dtype, seed=12)
    positions = torch.tensor(list(range(170, 300)) + list(range(77)), dtype=torch.int32, device=DEV)
    token_req = torch.tensor([0] * 130 + [1] * 77, dtype=torch.int32, device=DEV)
    q_start = torch.tensor([0, 130, T], dtype=torch.int32, device=DEV)
    slots = torch.tensor([1, 2], dtype=torch.int32, device=DEV)
    inv = plain.rope_inv_freq(rot_dim, 10000.0).float().to(DEV)
    cos = torch.empty(T, rot_dim // 2, device=DEV)
    sin = torch.empty(T, rot_dim // 2, device=DEV)
    ops.rope_table(cos, sin, positions, inv)
    assert ops.prefill_attention_rotates(rot_dim, interleaved)
    assert not ops.prefill_attention_rotates(32, False) and not ops.prefill_attention_rotates(16, True)
    kv_slot = torch.empty(T, dtype=torch.int32, device=DEV)
    ops.kv_slots(kv_slot, positions=positions, token_req=token_req, slots=slots, table=table,
                 page_size=page, num_pages=kc.shape[0])
    outs, caches = [], []
    for fused in (False, True):
        qkv, k2, v2 = qkv0.clone(), kc.clone(), vc.clone()
        ops.rope_kv_write(qkv, k2, v2, cos, sin, rot_dim=rot_dim, interleaved=interleaved, kv_slot=kv_slot,
                          nh=nh, nkv=nkv, d=d, rotate_q=not fused)
        if fused:
            assert torch.equal(qkv[:, :nh * d], qkv0[:, :nh * d])  # the queries were left alone
        out = torch.full((T, nh * d), float("nan"), dtype=dtype, device=DEV)
        extra = dict(cos=cos, sin=sin, rot_dim=rot_dim, interleaved=interleaved) if fused else {}
        ops.prefill_attention(out, qkv, k2, v2, table=table, positions=positions, q_start=q_start,
                              slots=slots, num_reqs=2, nh=nh, nkv=nkv, d=d, scale=d ** -0.5, nsplit=nsplit,
                              part_o=torch.empty(T * nh * nsplit, d, device=DEV),
                              part_ml=torch.empty(T * nh * nsplit, 2, device=DEV), **extra)
        outs.append(out)
        caches.append((k2, v2))
    assert not torch.isnan(outs[0]).any()
    assert torch.equal(outs[0], outs[1])
    assert torch.equal(caches[0][0].view(torch.int16), caches[1][0].view(torch.int16))  # the keys were rotated all the same
    with pytest.raises(ops.KernelError, match="rotary tables"):
        ops.prefill_attention(outs[0], qkv0, kc, vc, table=table, positions=positions, q_start=q_start,
                              slots=slots, num_reqs=2, nh=nh, nkv=nkv, d=d, scale=d ** -0.5,
                              cos=cos[:, :8].contiguous(), sin=sin[:, :8].contiguous(), rot_dim=16)


def test_decode_attention_says_what_it_does_not_serve(ops):
    assert not ops.prefill_attention_supported(4, 2, 96, 16, torch.bfloat16)
    assert not ops.prefill_attention_supported(4, 2, 64, 8, torch.bfloat16)
    assert not ops.prefill_attention_supported(4, 2, 64, 16, torch.float32)
    assert not ops.decode_attention_supported(4, 2, 48, 16, torch.bfloat16)   # head size not x32
    assert not ops.decode_attention_supported(4, 2, 64, 8, torch.bfloat16)    # page not x16
    assert not ops.decode_attention_supported(34, 2, 64, 16, torch.bfloat16)  # 17 heads a group
    assert not ops.decode_attention_supported(4, 2, 64, 16, torch.float32)


def test_paged_attention_refuses_unsupported_head_sizes(ops):
    from kvcore_amd.ops.library import KernelError

    kc, vc = make_cache(2, 1, 4, 24, torch.float32)
    q = rnd(1, 24)
    with pytest.raises(KernelError, match="multiple of 16"):
        ops.paged_attention(torch.empty(1, 24, device=DEV), q, kc, vc,
                            table=torch.zeros(1, 1, dtype=torch.int32, device=DEV),
                            positions=torch.zeros(1, dtype=torch.int32, device=DEV),
                            token_req=torch.zeros(1, dtype=torch.int32, device=DEV),
                            slots=torch.zeros(1, dtype=torch.int32, device=DEV),
                            nh=1, nkv=1, d=24, scale=1.0)


def test_table_update(ops):
    table = torch.zeros(3, 5, dtype=torch.int32, device=DEV)
    triples = torch.tensor([0, 0, 7, 2, 4, 9, 1, 3, 8, 5, 0, 1, 0, 9, 1], dtype=torch.int32, device=DEV)
    ops.table_update(table, triples, 5)  # the last two are outside the table and are dropped
    want = torch.zeros(3, 5, dtype=torch.int32)
    want[0, 0], want[2, 4], want[1, 3] = 7, 9, 8
    assert torch.equal(table.cpu(), want)


# -------------------------------------------------------------------------- sampling
def sample_rows(ops, logits, temps, top_k, top_p, seeds, index, workspace=None, filters=3):
    S = logits.shape[0]
    out = torch.empty(S, dtype=torch.int32, device=DEV)
    t = lambda v, dt: torch.tensor(v, dtype=dt, device=DEV)  # noqa: E731
    lo = [s & 0xFFFFFFFF for s in seeds]
    hi = [(s >> 32) & 0xFFFFFFFF for s in seeds]
    ops.sample(out, logits, temperature=t(temps, torch.float32), top_k=t(top_k, torch.int32),
               top_p=t(top_p, torch.float32), seed_lo=t(lo, torch.int64).to(torch.int32),
               seed_hi=t(hi, torch.int64).to(torch.int32), index=t(index, torch.int32),
               workspace=workspace, filters=filters)
    return out.cpu().tolist()


def test_argmax_takes_the_lowest_index_among_equals(ops):
    logits = rnd(4, 1000, seed=9)
    logits[1, 400] = logits[1, 17] = 50.0
    logits[2, 999] = 60.0
    out = torch.empty(4, dtype=torch.int32, device=DEV)
    ops.argmax(out, logits)
    want = logits.cpu().argmax(-1).tolist()
    want[1] = 17
    assert out.cpu().tolist() == want
    wide = torch.zeros(4, 1100, device=DEV)
    wide[:, :1000] = logits
    ops.argmax(out, wide[:, :1000])
    assert out.cpu().tolist() == want
    # long rows searched by several blocks: ties across chunk borders still go to the lowest index
    V = 3 * 8192 + 77
    long = rnd(5, V, seed=10)
    long[0, 8191] = long[0, 8192] = 70.0
    long[1, V - 1] = 70.0
    long[2, 0] = long[2, 20000] = 70.0
    part_val = torch.empty(5 * 4, device=DEV)
    part_idx = torch.empty(5 * 4, dtype=torch.int32, device=DEV)
    out5 = torch.empty(5, dtype=torch.int32, device=DEV)
    ops.argmax(out5, long, part_val, part_idx)
    want5 = long.cpu().argmax(-1).tolist()
    want5[0], want5[1], want5[2] = 8191, V - 1, 0
    assert out5.cpu().tolist() == want5
    ops.argmax(out5, long)
    assert out5.cpu().tolist() == want5


@pytest.mark.parametrize("V", [331, 5000])
def test_sample_matches_the_plain_sampler_draw_for_draw(ops, V):
    S = 24
    logits = rnd(S, V, scale=2.0, seed=V)
    temps = [0.0, 0.8, 1.0, 1.7] * 6
    top_k = [0, 0, 5, 40, 0, 3] * 4
    top_p = [1.0, 1.0, 1.0, 0.9, 0.5, 0.3] * 4
    seeds = [(12345 + 977 * i) | ((i * 31) << 32) for i in range(S)]
    index = [i * 3 for i in range(S)]
    got = sample_rows(ops, logits, temps, top_k, top_p, seeds, index)
    for i in range(S):
        want = plain_sampling.sample(logits[i].cpu(), temperature=temps[i], top_k=top_k[i] or None,
                                     top_p=top_p[i], seed=seeds[i], index=index[i])
        assert got[i] == want, f"row {i}: temperature {temps[i]} top_k {top_k[i]} top_p {top_p[i]}"
    # a row's draw does not depend on its batch-mates
    alone = sample_rows(ops, logits[5:6], temps[5:6], top_k[5:6], top_p[5:6], seeds[5:6], index[5:6])
    assert alone[0] == got[5]
    assert ops.sample_workspace_words(S, V) == 0  # rows this short stay with one block each


def test_sample_with_several_blocks_a_row_gives_the_same_draws(ops):
    """Long rows, each dealt to several blocks through a workspace (left dirty on purpose):
    the draws are those of one block a row and of the plain sampler, whatever passes the
    caller says are needed."""
    S, V = 12, 3 * 8192 + 77
    logits = rnd(S, V, scale=2.5, seed=3)
    logits[2, 8191] = logits[2, 8192] = 30.0  # equal largest values on either side of a chunk border
    temps = [0.0, 0.8, 1.0, 1.7] * 3
    top_k = [0, 0, 5, 400, 0, 3] * 2
    top_p = [1.0, 1.0, 1.0, 0.9, 0.5, 0.3] * 2
    seeds = [(999 + 131 * i) | ((i * 7) << 32) for i in range(S)]
    index = [i * 5 for i in range(S)]
    words = ops.sample_workspace_words(S, V)
    assert words > 0
    work = torch.full((words,), -1, dtype=torch.int64, device=DEV)
    one_block = sample_rows(ops, logits, temps, top_k, top_p, seeds, index)
    several = sample_rows(ops, logits, temps, top_k, top_p, seeds, index, workspace=work)
    assert several == one_block
    again = sample_rows(ops, logits, temps, top_k, top_p, seeds, index, workspace=work)  # a used workspace
    assert again == one_block
    for i in (0, 1, 2, 3, 4, 5, 9):
        want = plain_sampling.sample(logits[i].cpu(), temperature=temps[i], top_k=top_k[i] or None,
                                     top_p=top_p[i], seed=seeds[i], index=index[i])
        assert several[i] == want, f"row {i}"
    # rows without filters: the passes for them may be left out
    plain_rows = [0, 1, 6, 7]
    sub = lambda v: [v[i] for i in plain_rows]  # noqa: E731
    assert all(top_k[i] == 0 and top_p[i] == 1.0 for i in plain_rows)
    got = sample_rows(ops, logits[plain_rows], sub(temps), sub(top_k), sub(top_p), sub(seeds), sub(index),
                      workspace=work, filters=0)
    assert got == sub(one_block)
    # only top-k, only top-p
    for rows_, filt in (([2, 8], 1), ([4, 10], 2)):
        sub = lambda v: [v[i] for i in rows_]  # noqa: E731
        got = sample_rows(ops, logits[rows_], sub(temps), sub(top_k), sub(top_p), sub(seeds), sub(index),
                          workspace=work, filters=filt)
        assert got == sub(one_block)


def test_sample_follows_the_probabilities_and_top_k_top_p_vectors(ops):
    base = torch.tensor([1.0, 0.0, 2.0, -1.0, 0.5], device=DEV)
    n = 4000
    logits = base.repeat(n, 1)
    draws = sample_rows(ops, logits, [0.8] * n, [0] * n, [1.0] * n, [42] * n, list(range(n)))
    probs = torch.softmax(base.double().cpu() / 0.8, dim=0)
    counts = torch.bincount(torch.tensor(draws), minlength=5).double()
    chi2 = float(((counts - n * probs) ** 2 / (n * probs)).sum())
    assert chi2 < 18.5
    # the reference's vectors (tests/test_sampler.py:49-68): only kept entries are ever drawn
    k_logits = torch.tensor([[1.0, 2.0, 3.0, 4.0]], device=DEV).repeat(200, 1)
    got = set(sample_rows(ops, k_logits, [1.0] * 200, [2] * 200, [1.0] * 200, [1] * 200, list(range(200))))
    assert got == {2, 3}
    p_logits = torch.tensor([[10.0, 9.0, 0.0, -1.0]], device=DEV).repeat(200, 1)
    got = set(sample_rows(ops, p_logits, [1.0] * 200, [0] * 200, [0.8] * 200, [1] * 200, list(range(200))))
    assert got == {0, 1}


@pytest.mark.parametrize("M,H,I", [(1, 64, 48), (8, 4096, 1024), (16, 136, 200), (5, 4104, 88),
                                   (8, 2048, 512), (3, 512, 64)])
@pytest.mark.parametrize("with_bias", [False, True])
def test_norms_folded_into_the_products_around_them(ops, M, H, I, with_bias):
    """residual += x1 W1^T; x2 = rmsnorm(residual) * gain; y = silu(x2 Wg^T) * (x2 Wu^T), once
    with the norm as a kernel of its own and once folded into the two products."""
    eps = 1e-5
    x1 = rnd(M, I, dtype=torch.bfloat16, seed=1)
    w1 = rnd(H, I, dtype=torch.bfloat16, seed=2, scale=0.1)
    b1 = rnd(H, dtype=torch.bfloat16, seed=3) if with_bias else None
    w2 = rnd(2 * I, H, dtype=torch.bfloat16, seed=4, scale=0.05)
    b2 = rnd(2 * I, dtype=torch.bfloat16, seed=5) if with_bias else None
    w3 = rnd(I, H, dtype=torch.bfloat16, seed=6, scale=0.05)
    gain = (1 + 0.1 * rnd(H, dtype=torch.float32, seed=7))
    residual0 = 3 * rnd(M, H, dtype=torch.float32, seed=8)

    # folded
    res = residual0.clone()
    rows = torch.full((M, H), float("nan"), dtype=torch.bfloat16, device=DEV)
    parts = torch.full((16, -(-H // 16)), float("nan"), device=DEV)
    scaled = ops.linear(ops.ResidualSink(res, gain, eps, rows, parts), x1, w1, b1)
    assert isinstance(scaled, ops.ScaledRows) and scaled.ss_parts.shape == (M, ops.skinny_blocks(H, I))
    y = torch.full((M, I), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.linear_silu_mul(y, scaled, w2, b2, None)
    z = torch.full((M, I), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.linear(z, scaled, w3)

    # the formula in float64
    r = residual0.double() + x1.double() @ w1.double().T + (b1.double() if with_bias else 0.0)
    assert torch.allclose(res.double(), r, atol=1e-4, rtol=1e-5)
    assert torch.allclose(scaled.ss_parts.double().sum(1), (r * r).sum(1), rtol=1e-5)
    x2 = plain.rms_norm(r, gain.double(), eps)
    want_y = plain.silu_and_mul(x2 @ w2.double().T + (b2.double() if with_bias else 0.0))
    want_z = x2 @ w3.double().T
    def close(got, want):  # bfloat16 activations: each element within 2% of the row's scale
        err = (got.double() - want).abs()
        return bool((err <= 2e-2 * want.abs().amax(dim=1, keepdim=True) + 1e-3).all()) and \
            float(err.norm() / want.norm()) < 1e-2

    assert close(y, want_y)
    assert close(z, want_z)

    # and the unfolded kernels agree with the folded ones to bfloat16 rounding
    res2 = residual0.clone()
    delta = torch.empty(M, H, dtype=torch.bfloat16, device=DEV)
    ops.linear(delta, x1, w1, b1)
    x2b = torch.empty(M, H, dtype=torch.bfloat16, device=DEV)
    ops.add_rmsnorm(x2b, res2, delta, gain, eps)
    z2 = torch.empty(M, I, dtype=torch.bfloat16, device=DEV)
    ops.linear(z2, x2b, w3)
    assert close(z, z2.double())


@pytest.mark.parametrize("M,N,K", [(64, 4096, 14336), (24, 6144, 4096), (48, 4096, 4096), (33, 1024, 8192)])
def test_library_product_inside_a_graph_replays_right(ops, M, N, K):
    """Steps of more than 16 rows use the vendor matrix product, also inside captured graphs
    (some of its kernels split K over blocks and need a workspace).  Every replay, with other
    work between, must give the bits of the call outside a graph."""
    w = rnd(N, K, dtype=torch.bfloat16, seed=1, scale=0.05)
    x = rnd(M, K, dtype=torch.bfloat16, seed=2)
    out = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    ops.linear(out, x, w)
    want = out.clone()
    assert torch.allclose(want.double(), x.double() @ w.double().T, atol=0.3, rtol=3e-2)
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        ops.linear(out, x, w)  # warm-up on the capturing stream
        stream.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            ops.linear(out, x, w)
    torch.cuda.current_stream().wait_stream(stream)
    other = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    for i in range(4):
        out.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), f"replay {i}"
        ops.linear(other, rnd(M, K, dtype=torch.bfloat16, seed=10 + i), w)  # eager work between
        torch.cuda.synchronize()


@pytest.mark.parametrize("nsplit", [1, 7, 32])
def test_decode_attention_long_context(ops, nsplit):
    """Twenty thousand keys: many blocks a wave, a wide block table, many parts."""
    dtype = torch.bfloat16
    nh, nkv, d, page = 8, 2, 128, 16
    seq_lens = [20000, 4099, 1]
    R = len(seq_lens)
    kc, vc, table, dense = paged_setup(seq_lens, nkv, d, page, dtype, seed=3)
    q = rnd(R, nh * d, dtype=dtype, seed=4)
    positions = torch.tensor([n - 1 for n in seq_lens], dtype=torch.int32, device=DEV)
    token_req = torch.arange(R, dtype=torch.int32, device=DEV)
    slots = torch.arange(1, R + 1, dtype=torch.int32, device=DEV)
    out = torch.full((R, nh * d), float("nan"), dtype=dtype, device=DEV)
    part_o = torch.full((R * nh * nsplit, d), float("nan"), device=DEV)
    part_ml = torch.full((R * nh * nsplit, 2), float("nan"), device=DEV)
    scale = d ** -0.5
    ops.decode_attention(out, q, kc, vc, table=table, positions=positions, token_req=token_req,
                         slots=slots, nh=nh, nkv=nkv, d=d, scale=scale, nsplit=nsplit,
                         part_o=part_o, part_ml=part_ml)
    got = out.double().cpu().view(R, nh, d)
    qd = q.double().cpu().view(R, nh, d)
    for r, n in enumerate(seq_lens):
        k, v = dense[r][0].double(), dense[r][1].double()  # [n, nkv, d]
        for h in range(nh):
            p = torch.softmax((k[:, h // (nh // nkv)] @ qd[r, h]) * scale, dim=0)
            want = p @ v[:, h // (nh // nkv)]
            assert torch.allclose(got[r, h], want, atol=1e-2, rtol=1e-2), (n, h)


@pytest.mark.parametrize("nh,nkv,d,whole,nsplit", [(8, 2, 128, 2100, 1), (8, 1, 64, 2100, 1), (32, 8, 128, 4200, 1),
                                                   (8, 2, 128, 2100, 7), (8, 1, 64, 2100, 2),
                                                   (16, 4, 128, 2100, 1), (16, 4, 128, 3100, 1),
                                                   (12, 6, 128, 2100, 1), (16, 4, 64, 4200, 1)])
def test_prefill_attention_long_context_and_many_tokens(ops, nh, nkv, d, whole, nsplit):
    """A portion of 700 tokens after 6,000 others, and a whole prompt of thousands of tokens:
    hundreds of key tiles; the third case has enough tokens and kv heads that the kernel takes
    its larger query tiles, the fourth and fifth deal each tile's keys to several blocks, and
    the last four take blocks of eight waves (one tile a block, a late and an early tile a
    block, six kv heads, which the eight dies do not share out evenly, and heads of 64 with
    their tiles of 128 keys)."""
    dtype, page = torch.bfloat16, 16
    seq_lens = [6700, whole]
    q_lens = [700, whole]
    kc, vc, table, dense = paged_setup(seq_lens, nkv, d, page, dtype, seed=5)
    T = sum(q_lens)
    q = rnd(T, nh * d, dtype=dtype, seed=6)
    positions = torch.tensor(list(range(6000, 6700)) + list(range(whole)), dtype=torch.int32, device=DEV)
    q_start = torch.tensor([0, 700, 700 + whole], dtype=torch.int32, device=DEV)
    slots = torch.tensor([1, 2], dtype=torch.int32, device=DEV)
    out = torch.full((T, nh * d), float("nan"), dtype=dtype, device=DEV)
    scale = d ** -0.5
    ops.prefill_attention(out, q, kc, vc, table=table, positions=positions, q_start=q_start,
                          slots=slots, num_reqs=2, nh=nh, nkv=nkv, d=d, scale=scale, nsplit=nsplit,
                          part_o=torch.empty(T * nh * nsplit, d, device=DEV),
                          part_ml=torch.empty(T * nh * nsplit, 2, device=DEV))
    assert not torch.isnan(out).any()
    got = out.double().cpu().view(T, nh, d)
    qd = q.double().cpu().view(T, nh, d)
    g = nh // nkv
    for t in [0, 1, 15, 16, 333, 699, 700, 701, 731, 732, 1500, T - 1]:  # rows at tile edges and inside
        r = 0 if t < 700 else 1
        pos = int(positions[t])
        k, v = dense[r][0].double()[: pos + 1], dense[r][1].double()[: pos + 1]
        for h in (0, nh - 1):
            p = torch.softmax((k[:, h // g] @ qd[t, h]) * scale, dim=0)
            assert torch.allclose(got[t, h], p @ v[:, h // g], atol=1e-2, rtol=1e-2), (t, h)


def test_measured_peaks_are_of_this_chips_order(ops):
    """The benchmark's second yardstick: a kernel that only reads and one that only multiplies.
    An MI355X's data sheet says 8 TB/s and 2.5 PFLOP/s; the kernels must come within a factor
    of two of those and cannot exceed them."""
    peaks = ops.measure_peaks(DEV)
    assert 4e12 < peaks["read_bytes_per_s"] < 8.2e12, peaks
    assert 1.25e15 < peaks["mfma_bf16_flops_per_s"] < 2.6e15, peaks
