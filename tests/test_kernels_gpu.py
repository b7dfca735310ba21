"""Each HIP kernel alone against its plain torch reference (tests/torch_ops.py), at sizes
other than the engine configurations': widths and vocabularies that are no power of two,
head sizes in steps of 16, odd head counts."""
import types

import pytest
import torch

from tests.torch_ops import TorchOps

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    from return_amd.kernels.hip_ops import HipOps
    return HipOps(DEV)


@pytest.fixture(scope="module")
def ref():
    return TorchOps(DEV)


def tol(dtype):
    return dict(atol=2e-5, rtol=2e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)


def rnd(*shape, dtype=torch.float32, seed=0, scale=1.0):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


DTYPES = [torch.float32, torch.bfloat16]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("V,H,T", [(331, 120, 7), (1000, 4096, 3), (97, 100, 5), (500, 2560, 9), (64, 5120, 2)])
def test_embed(ops, ref, dtype, V, H, T):
    table = rnd(V, H, dtype=dtype)
    ids = torch.randint(0, V, (T,), dtype=torch.int32, device=DEV)
    a = torch.empty(T, H, dtype=torch.float32, device=DEV)
    b = torch.empty_like(a)
    ops.embed(table, ids, a)
    ref.embed(table, ids, b)
    assert torch.equal(a, b)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("R,H", [(5, 120), (33, 1000), (3, 5120)])
@pytest.mark.parametrize("mode", ["plain", "delta", "rows", "delta_rows"])
def test_add_rmsnorm(ops, ref, dtype, R, H, mode):
    h = rnd(R, H, seed=1, scale=3.0)
    delta = rnd(R, H, dtype=dtype, seed=2) if "delta" in mode else None
    rows = torch.tensor([R - 1, 0, R // 2], dtype=torch.int32, device=DEV) if "rows" in mode else None
    w = 1.0 + 0.1 * rnd(H, seed=3)
    M = R if rows is None else 3
    ha, hb = h.clone(), h.clone()
    a = torch.empty(M, H, dtype=dtype, device=DEV)
    b = torch.empty_like(a)
    ops.add_rmsnorm(ha, delta, w, 1e-5, a, rows)
    ref.add_rmsnorm(hb, delta, w, 1e-5, b, rows)
    torch.testing.assert_close(a.float(), b.float(), **tol(dtype))
    torch.testing.assert_close(ha, hb, atol=1e-6, rtol=1e-6)
    if rows is not None:
        assert torch.equal(ha, h)          # with a row list the residual stream is left alone


@pytest.mark.parametrize("dtype", DTYPES)
def test_rmsnorm_mean_square_is_one(ops, dtype):
    """With weight 1 the output row has mean square 1/(1 + eps/ms): the norm divides by the RMS."""
    h = rnd(4, 777, seed=5, scale=7.0)
    w = torch.ones(777, device=DEV)
    out = torch.empty(4, 777, dtype=dtype, device=DEV)
    ops.add_rmsnorm(h, None, w, 1e-6, out, None)
    ms = (out.float() ** 2).mean(-1)
    torch.testing.assert_close(ms, torch.ones_like(ms), atol=1e-2 if dtype == torch.bfloat16 else 1e-5, rtol=0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("D", [16, 48, 80, 128, 256])
def test_head_rmsnorm_and_rope(ops, ref, dtype, D):
    T, heads = 9, 5
    x = rnd(T, heads, D, dtype=dtype, seed=D)
    w = 1.0 + 0.1 * rnd(D, seed=7)
    a, b = x.clone(), x.clone()
    ops.head_rmsnorm(a, w, 1e-6)
    ref.head_rmsnorm(b, w, 1e-6)
    torch.testing.assert_close(a.float(), b.float(), **tol(dtype))
    for R in (D, D // 2 if (D // 2) % 2 == 0 else D):
        pos = torch.tensor([0, 1, 2, 100, 299, 7, 8, 9, 10], dtype=torch.int32, device=DEV)
        ang = torch.outer(torch.arange(300, dtype=torch.float32), 1.0 / (10000.0 ** (torch.arange(0, R // 2).float() / (R // 2))))
        cos, sin = ang.cos().to(DEV), ang.sin().to(DEV)
        a, b = x.clone(), x.clone()
        ops.rope(a, pos, cos, sin, R)
        ref.rope(b, pos, cos, sin, R)
        torch.testing.assert_close(a.float(), b.float(), **tol(dtype))
        assert torch.equal(a[0], x[0])     # position 0 is the identity


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("Hq,Hkv,D,R,norm", [(4, 2, 16, 16, True), (6, 1, 32, 32, True), (5, 5, 48, 48, True),
                                           (3, 1, 80, 32, False), (8, 2, 128, 128, True),
                                           (2, 2, 256, 64, True), (1, 1, 512, 512, True),
                                           (7, 1, 80, 80, True), (2, 1, 192, 192, False), (3, 1, 64, 0, True),
                                           (9, 3, 256, 256, True),
                                           # head sizes that are no multiple of 16, or beyond 256: the general kernel
                                           (3, 1, 24, 24, True), (4, 2, 40, 40, True), (5, 1, 72, 36, True),
                                           (2, 1, 320, 320, True), (3, 3, 6, 6, True), (2, 2, 130, 130, False)])
def test_qkv_prepare(ops, ref, dtype, Hq, Hkv, D, R, norm):
    T, P, pages = 11, 8, 6
    qkv = rnd(T, (Hq + 2 * Hkv) * D, dtype=dtype, seed=11)
    wq = 1.0 + 0.1 * rnd(D, seed=12) if norm else None
    wk = 1.0 + 0.1 * rnd(D, seed=13) if norm else None
    pos = torch.arange(20, 20 + T, dtype=torch.int32, device=DEV)
    ang = torch.outer(torch.arange(64, dtype=torch.float32), 1.0 / (1e6 ** (torch.arange(0, R // 2).float() / (R // 2))))
    cos, sin = ang.cos().to(DEV), ang.sin().to(DEV)
    slots = torch.randperm(P * pages)[:T].to(torch.int32).to(DEV)
    outs = []
    for o in (ops, ref):
        q = torch.zeros(T, Hq, D, dtype=dtype, device=DEV)
        kp = torch.zeros(pages, Hkv, P, D, dtype=dtype, device=DEV)
        vp = torch.zeros_like(kp)
        o.qkv_prepare(qkv, Hq, Hkv, D, wq, wk, 1e-6, pos, cos, sin, R, q, kp, vp, slots)
        outs.append((q, kp, vp))
    for a, b in zip(*outs):
        torch.testing.assert_close(a.float(), b.float(), **tol(dtype))
    # without pools nothing is written and q is the same
    q2 = torch.zeros(T, Hq, D, dtype=dtype, device=DEV)
    ops.qkv_prepare(qkv, Hq, Hkv, D, wq, wk, 1e-6, pos, cos, sin, R, q2, None, None, slots)
    assert torch.equal(q2, outs[0][0])


@pytest.mark.parametrize("dtype", DTYPES)
def test_split_and_kv_write(ops, ref, dtype):
    T, Hq, Hkv, D, P, pages = 6, 3, 2, 48, 4, 5
    qkv = rnd(T, (Hq + 2 * Hkv) * D, dtype=dtype, seed=21)
    slots = torch.randperm(P * pages)[:T].to(torch.int32).to(DEV)
    res = []
    for o in (ops, ref):
        q = torch.empty(T, Hq, D, dtype=dtype, device=DEV)
        k = torch.empty(T, Hkv, D, dtype=dtype, device=DEV)
        v = torch.empty_like(k)
        o.split_heads(qkv, Hq, Hkv, D, q, k, v)
        kp = torch.zeros(pages, Hkv, P, D, dtype=dtype, device=DEV)
        vp = torch.zeros_like(kp)
        o.kv_write(k, v, kp, vp, slots)
        res.append((q, k, v, kp, vp))
    for a, b in zip(*res):
        assert torch.equal(a, b)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,I", [(3, 200), (17, 1111)])
def test_silu_mul(ops, ref, dtype, T, I):
    gu = rnd(T, 2 * I, dtype=dtype, seed=31, scale=3.0)
    a = torch.empty(T, I, dtype=dtype, device=DEV)
    b = torch.empty_like(a)
    ops.silu_mul(gu, a)
    ref.silu_mul(gu, b)
    torch.testing.assert_close(a.float(), b.float(), **tol(dtype))


@pytest.mark.parametrize("dtype,out_dtype", [(torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16),
                                             (torch.bfloat16, torch.float32)])
@pytest.mark.parametrize("M,N,K", [(1, 331, 120), (7, 100, 77), (64, 64, 64), (65, 129, 250), (200, 48, 1000)])
def test_linear(ops, monkeypatch, dtype, out_dtype, M, N, K):
    x = rnd(M, K, dtype=dtype, seed=41)
    w = rnd(N, K, dtype=dtype, seed=42, scale=0.1)
    want = x.double() @ w.double().t()
    for own in (False, True):               # the library's product where it is used, and the hand-written one
        monkeypatch.setattr(ops, "own_gemm", own)
        y = ops.linear(x, w, out_dtype=out_dtype)
        assert y.dtype == out_dtype and tuple(y.shape) == (M, N)
        if out_dtype == torch.float32:
            torch.testing.assert_close(y.double(), want, atol=2e-5 * K ** 0.5, rtol=1e-5)
        else:
            torch.testing.assert_close(y.double(), want, atol=3e-2, rtol=2e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,I,K", [(1, 160, 96), (3, 200, 120), (8, 1000, 256), (20, 48, 64), (8, 24, 40)])
def test_linear_silu_mul(ops, ref, dtype, M, I, K):
    x = rnd(M, K, dtype=dtype, seed=43)
    w = rnd(2 * I, K, dtype=dtype, seed=44, scale=0.2)
    a, b = ops.linear_silu_mul(x, w), ref.linear_silu_mul(x, w)
    assert a.shape == (M, I)
    torch.testing.assert_close(a.float(), b.float(), **tol(dtype))


@pytest.mark.parametrize("M", [1, 5, 16, 17, 40, 64])
@pytest.mark.parametrize("N,K", [(331, 120), (48, 1000), (1000, 264)])
def test_skinny_product_fp32_out(ops, M, N, K):
    """bf16 rows times bf16 weights with fp32 results (the output head's product)."""
    x = rnd(M, K, dtype=torch.bfloat16, seed=45)
    w = rnd(N, K, dtype=torch.bfloat16, seed=46, scale=0.1)
    y = ops.linear(x, w, out_dtype=torch.float32)
    torch.testing.assert_close(y.double(), x.double() @ w.double().t(), atol=1e-4 * K ** 0.5, rtol=1e-5)


@pytest.mark.parametrize("M", [1, 2, 7, 8, 9, 16])
@pytest.mark.parametrize("N,K,grid", [(331, 120, 0), (1000, 264, 7), (48, 4096, 0), (6200, 72, 512)])
def test_resident_product(ops, ref, M, N, K, grid):
    """The product with x resident in LDS, called directly: bf16 and fp32 results, the gated
    form, more tiles than workgroups, widths that are no multiple of the tile."""
    from return_amd.kernels.hip_ops import _code, _ptr
    st = torch.cuda.current_stream().cuda_stream
    x = rnd(M, K, dtype=torch.bfloat16, seed=3)
    w = rnd(2 * N, K, dtype=torch.bfloat16, seed=4) * 0.2
    want = x.double() @ w.double().t()
    for out_dtype in (torch.bfloat16, torch.float32):
        y = torch.full((M, N), 7.0, dtype=out_dtype, device=DEV)
        assert ops.lib.ra_gemm_resident_bf16(_ptr(x), _ptr(w), _ptr(y), M, N, K, 0, _code(out_dtype), grid, st) == 0
        if out_dtype == torch.float32:
            torch.testing.assert_close(y.double(), want[:, :N], atol=1e-4 * K ** 0.5, rtol=1e-5)
        else:
            torch.testing.assert_close(y.float(), want[:, :N].float(), **tol(torch.bfloat16))
    y = torch.full((M, N), 7.0, dtype=torch.bfloat16, device=DEV)
    assert ops.lib.ra_gemm_resident_bf16(_ptr(x), _ptr(w), _ptr(y), M, N, K, 1, _code(torch.bfloat16), grid, st) == 0
    g, u = want[:, :N], want[:, N:]
    torch.testing.assert_close(y.float(), (g * torch.sigmoid(g) * u).float(), **tol(torch.bfloat16))
    # what does not fit is refused, not computed
    assert ops.lib.ra_gemm_resident_bf16(_ptr(x), _ptr(w), _ptr(y), 17, N, K, 0, _code(torch.bfloat16), grid, st) != 0
    assert not ops.lib.ra_gemm_resident_fits(16, 8192, 0) and ops.lib.ra_gemm_resident_fits(8, 8192, 0)


@pytest.mark.parametrize("gated", [False, True])
@pytest.mark.parametrize("N,K", [(6144, 4096), (2500, 2560), (700, 4096), (4099, 520), (37, 64), (4096, 12288), (300, 9728),
                                 (5200, 4104), (1100, 5120), (300, 8192), (5120, 12288), (15000, 8200)])
def test_product_that_sweeps_the_weight(ops, N, K, gated):
    """The product that reads W as one sweep (column c with workgroup c % CUs): widths that fill
    every wave's 512 columns and widths that leave waves idle, widths of several spans of 4,096 (whole
    ones and one that ends after 8 columns; up to two spans x stays in registers, beyond it is read
    per span, and once for all tiles where a workgroup has two to four of them), column counts that are no multiple of
    the workgroups or of a tile, fewer columns than workgroups, 1 to 32 rows, both result types, the
    gated form; and what it does not take is refused."""
    from return_amd.kernels.hip_ops import _code, _ptr
    lib, st = ops.lib, torch.cuda.current_stream().cuda_stream
    w = rnd((2 if gated else 1) * N, K, dtype=torch.bfloat16, seed=N, scale=0.05)
    for M in (1, 2, 5, 8, 13, 16) + ((17, 24, 32) if K <= 4096 else ()):
        x = rnd(M, K, dtype=torch.bfloat16, seed=M + 1)
        want = x.double() @ w.double().t()
        if gated:
            g, u = want[:, :N], want[:, N:]
            want = g * torch.sigmoid(g) * u
        for out_dtype in ((torch.bfloat16,) if gated else (torch.bfloat16, torch.float32)):
            for grid in (ops.cu_count, 7):
                y = torch.full((M, N), 9.0, dtype=out_dtype, device=DEV)
                assert lib.ra_gemm_sweep_bf16(_ptr(x), _ptr(w), _ptr(y), M, N, K, int(gated), _code(out_dtype), grid, st) == 0
                if out_dtype == torch.float32:
                    torch.testing.assert_close(y.double(), want, atol=1e-4 * K ** 0.5, rtol=1e-5)
                else:
                    torch.testing.assert_close(y.float(), want.float(), **tol(torch.bfloat16))
    too_many = 33 if K <= 4096 else 17
    y = torch.empty(too_many, N, dtype=torch.bfloat16, device=DEV)
    x = rnd(too_many, K, dtype=torch.bfloat16)
    assert lib.ra_gemm_sweep_bf16(_ptr(x), _ptr(w), _ptr(y), too_many, N, K, int(gated), _code(torch.bfloat16), 256, st) != 0
    assert lib.ra_gemm_sweep_fits(8, 4104) and not lib.ra_gemm_sweep_fits(8, 4100) and lib.ra_gemm_sweep_fits(16, 32768)
    assert not lib.ra_gemm_sweep_fits(8, 32776) and lib.ra_gemm_sweep_fits(32, 4096) and not lib.ra_gemm_sweep_fits(17, 4104)
    if gated:
        assert lib.ra_gemm_sweep_bf16(_ptr(x), _ptr(w), _ptr(y), 8, N, K, 1, _code(torch.float32), 256, st) != 0


@pytest.mark.parametrize("N,K", [(331, 120), (1000, 264), (48, 4096)])
def test_every_way_to_form_a_product(ops, monkeypatch, N, K):
    """linear and linear_silu_mul under every way the plan may name, at every measured row count:
    whatever the measurement at load time picks, the product is the product."""
    plan = {}
    monkeypatch.setattr(ops, "product_plan", plan)
    w = rnd(2 * N, K, dtype=torch.bfloat16, seed=4, scale=0.2)
    ways = set()
    for M in (1, 3, 8, 11, 16, 33, 64):
        x = rnd(M, K, dtype=torch.bfloat16, seed=M)
        want = x.double() @ w.double().t()
        for out_dtype in (torch.bfloat16, torch.float32):
            for how in ops._candidates(M, 2 * N, K, False, out_dtype):
                plan.clear()
                plan[(ops._rows_step(M), 2 * N, K, False, out_dtype)] = how
                assert ops.route_linear(M, 2 * N, K, out_dtype) == how
                y = ops.linear(x, w, out_dtype=out_dtype)
                assert y.dtype == out_dtype
                if out_dtype == torch.float32:
                    torch.testing.assert_close(y.double(), want, atol=1e-4 * K ** 0.5, rtol=1e-5)
                else:
                    torch.testing.assert_close(y.float(), want.float(), **tol(torch.bfloat16))
                ways.add(how)
        g, u = want[:, :N], want[:, N:]
        for how in ops._candidates(M, N, K, True, torch.bfloat16):
            plan.clear()
            plan[(ops._rows_step(M), N, K, True, torch.bfloat16)] = how
            y = ops.linear_silu_mul(x, w)
            torch.testing.assert_close(y.float(), (g * torch.sigmoid(g) * u).float(), **tol(torch.bfloat16))
            ways.add("gated " + how)
    assert {"library", "skinny", "resident256", "resident512", "sweep", "gated two", "gated skinny",
            "gated resident512", "gated sweep"} <= ways


@pytest.mark.parametrize("M", [1, 7, 16])
@pytest.mark.parametrize("H,K1,N2", [(512, 264, 331), (4096, 4096, 1000), (1024, 12288, 760), (264, 520, 4500),
                                     (640, 8192, 300), (5120, 5120, 520), (6000, 8200, 264)])
def test_norm_finished_inside_the_products_around_it(ops, ref, M, H, K1, N2):
    """h += x W1^T inside the product, the rows of the norm that follows left unfinished, and the
    products after it that finish them (plain, fp32 results, gated): against the residual addition,
    the norm and the products one after the other. K1 within one span of the sweep and beyond it, a
    width that is no multiple of the workgroups, more and fewer columns than workgroups."""
    from return_amd.parts.runtime import ScaledRows
    x = rnd(M, K1, dtype=torch.bfloat16, seed=1)
    w1 = rnd(H, K1, dtype=torch.bfloat16, seed=2, scale=0.05)
    w2 = rnd(2 * N2, H, dtype=torch.bfloat16, seed=3, scale=0.05)
    wn = 1.0 + 0.2 * rnd(H, seed=4)
    h0 = rnd(M, H, seed=5, scale=2.0)
    eps = 1e-5
    assert ops.can_defer_norm(M, w1, w2, True) and ops.can_defer_norm(M, w1, w2, False)
    h = h0.clone()
    rows = ops.linear_add_norm(x, w1, h, wn, eps)
    assert isinstance(rows, ScaledRows) and rows.partials.shape[0] == M and rows.size == H
    # the residual stream: h0 + bf16(x W1^T)
    delta = (x.double() @ w1.double().t())
    torch.testing.assert_close(h.double(), h0.double() + delta, atol=2e-2, rtol=2e-2)
    want_h = h.double()                                     # from here on with the h the kernel made
    torch.testing.assert_close(rows.tensor.float(), (want_h * wn.double()).float(), **tol(torch.bfloat16))
    torch.testing.assert_close(rows.partials.double().sum(-1), (want_h * want_h).sum(-1), atol=1e-3, rtol=1e-4)
    xn = want_h * (1.0 / torch.sqrt((want_h * want_h).mean(-1, keepdim=True) + eps)) * wn.double()
    torch.testing.assert_close(ops.linear(rows, w2).float(), (xn @ w2.double().t()).float(), **tol(torch.bfloat16))
    # the products after it, exactly: from the operand as the kernel left it (rounded to bfloat16)
    xn = rows.tensor.double() * (1.0 / torch.sqrt((want_h * want_h).mean(-1, keepdim=True) + eps))
    y = xn @ w2.double().t()
    torch.testing.assert_close(ops.linear(rows, w2).float(), y.float(), **tol(torch.bfloat16))
    torch.testing.assert_close(ops.linear(rows, w2, out_dtype=torch.float32).double(), y, atol=3e-2, rtol=2e-2)
    g, u = y[:, :N2], y[:, N2:]
    torch.testing.assert_close(ops.linear_silu_mul(rows, w2).float(), (g * torch.sigmoid(g) * u).float(),
                               **tol(torch.bfloat16))
    # and a second residual product on unfinished rows (x itself ScaledRows)
    w3 = rnd(H, H, dtype=torch.bfloat16, seed=6, scale=0.05)
    h2 = h.clone()
    rows2 = ops.linear_add_norm(rows, w3, h2, wn, eps)
    # (what is added is the product rounded to bfloat16: half an ulp of it, 2^-8 of its size, and the sums' own error)
    added = xn @ w3.double().t()
    assert ((h2.double() - want_h - added).abs() <= added.abs() * 2.0 ** -8 + 2e-3).all()
    assert rows2.tensor.shape == (M, H)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("R,H,S", [(5, 120, 2), (33, 1000, 4), (64, 4096, 8), (9, 5120, 4), (7, 8192, 8), (3, 8200, 2)])
def test_add_rmsnorm_takes_a_product_in_shares(ops, ref, dtype, R, H, S):
    """The norm adds the shares of a product up in order, rounds the sum as the one product's result
    would have been rounded, and goes on as with that result; all rows, and a list of rows."""
    from return_amd.parts.runtime import Slabs
    shares = Slabs(rnd(S, R, H, seed=8))
    total = torch.zeros(R, H, device=DEV)
    for i in range(S):                                      # in order, as the kernel adds them
        total = total + shares.tensor[i]
    delta = total.to(dtype)
    w = 1.0 + 0.1 * rnd(H, seed=3)
    for rows in (None, torch.tensor([R - 1, 0, R // 2], dtype=torch.int32, device=DEV)):
        M = R if rows is None else 3
        ha, hb = rnd(R, H, seed=1, scale=3.0), rnd(R, H, seed=1, scale=3.0)
        a = torch.empty(M, H, dtype=dtype, device=DEV)
        b = torch.empty_like(a)
        ops.add_rmsnorm(ha, shares, w, 1e-5, a, rows)
        ref.add_rmsnorm(hb, delta, w, 1e-5, b, rows)
        torch.testing.assert_close(a.float(), b.float(), **tol(dtype))
        torch.testing.assert_close(ha, hb, atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("M", [8, 17, 64, 200, 600])
def test_product_for_the_residual_stream_in_every_form(ops, monkeypatch, M):
    """linear_residual under every way the plan may name: bfloat16 rows or shares whose sum is the product."""
    from return_amd.parts.runtime import Slabs
    plan = {}
    monkeypatch.setattr(ops, "product_plan", plan)
    N, K = 520, 1024
    x, w = rnd(M, K, dtype=torch.bfloat16, seed=M), rnd(N, K, dtype=torch.bfloat16, seed=4, scale=0.2)
    want = x.double() @ w.double().t()
    ways = ops._candidates(M, N, K, False, "residual")
    assert ("split4" in ways) == (M > 16) and "library" in ways
    for how in ways:
        plan.clear()
        plan[(ops._rows_step(M, True), N, K, False, "residual")] = how
        y = ops.linear_residual(x, w)
        if how.startswith("split"):
            assert isinstance(y, Slabs) and tuple(y.tensor.shape) == (int(how[5:]), M, N) and y.tensor.dtype == torch.float32
            torch.testing.assert_close(y.tensor.double().sum(0), want, atol=1e-3, rtol=1e-4)
        else:
            torch.testing.assert_close(y.float(), want.float(), **tol(torch.bfloat16))
    plan.clear()
    # the rule: many columns of K against few of N, 17 to 64 rows
    assert ops.route_linear(64, 4096, 12288, "residual") == "split4" and ops.route_linear(16, 4096, 12288, "residual") != "split4"
    assert not ops.route_linear(64, 4096, 4096, "residual").startswith("split")


def test_norms_are_not_deferred_where_the_sweep_does_not_form_the_products(ops, monkeypatch):
    bf = torch.bfloat16
    w1, w2 = rnd(512, 264, dtype=bf), rnd(300, 512, dtype=bf)
    assert ops.can_defer_norm(16, w1, w2, False)
    assert not ops.can_defer_norm(17, w1, w2, False)                    # more rows than the residual epilogue takes
    assert not ops.can_defer_norm(4, rnd(512, 260, dtype=bf), w2, False)   # K no multiple of 8
    assert not ops.can_defer_norm(4, w1.float(), w2.float(), False)     # float32: the plain kernels
    assert not ops.can_defer_norm(4, rnd(100, 264, dtype=bf), rnd(300, 100, dtype=bf), False)   # narrower than the chip
    assert not ops.can_defer_norm(4, w1, rnd(300, 520, dtype=bf), False)   # widths that do not meet
    # where a pair has been measured at load, the measurement decides
    monkeypatch.setattr(ops, "_defer", {(4, (512, 264), (300, 512), False): False})
    assert not ops.can_defer_norm(4, w1, w2, False) and ops.can_defer_norm(16, w1, w2, False)


def test_norm_pairs_are_measured_at_load(ops, monkeypatch):
    """tune_norm_pairs times every pair of products with a norm between them both ways, at the row counts
    up to 16, once in a process, and can_defer_norm follows what it found."""
    import return_amd.kernels.hip_ops as ho
    monkeypatch.setattr(ops, "_defer", {})
    monkeypatch.setattr(ho, "_NORM_PAIRS_MEASURED", {})
    bf = torch.bfloat16
    pairs = [(rnd(512, 264, dtype=bf, seed=i), 1.0 + 0.1 * rnd(512, seed=9), 1e-5, rnd(600, 512, dtype=bf, seed=20 + i), True)
             for i in range(3)]
    ops.tune_norm_pairs(pairs, max_rows=5)
    assert set(ops._defer) == {(r, (512, 264), (600, 512), True) for r in (1, 2, 4, 8)}
    assert all(isinstance(v, bool) for v in ops._defer.values())
    for (r, _, _, _), v in ops._defer.items():
        assert ops.can_defer_norm(r, pairs[0][0], pairs[0][3], True) == v
    calls = []
    monkeypatch.setattr(ops, "_time_over", lambda *a: calls.append(a) or 1.0)
    ops.tune_norm_pairs(pairs, max_rows=5)
    assert not calls                                                       # nothing is measured twice


def test_products_are_measured_once_and_the_plan_is_followed(ops, monkeypatch):
    """tune_products measures every shape at every row count up to the limit, once in a process, and
    notes only ways that exist; a measured choice is what route_* returns from then on; a kernel
    set that has not tuned follows the rules."""
    from return_amd.kernels.hip_ops import HipOps
    plan, measured = {}, {}
    monkeypatch.setattr(ops, "product_plan", plan)
    monkeypatch.setattr(ops, "_measured", measured)
    ws = [rnd(768, 256, dtype=torch.bfloat16, seed=i, scale=0.1) for i in range(3)]
    head = rnd(1000, 256, dtype=torch.bfloat16, seed=9, scale=0.1)
    products = [(w, True, None) for w in ws] + [(w, False, None) for w in ws] + [(head, False, torch.float32)]
    ops.tune_products(products, max_rows=5)
    steps = [r for r in ops.ROW_STEPS if r <= 8]                     # 5 rows are served by the step of 8
    assert set(measured) == {(r, 384, 256, True, torch.bfloat16) for r in steps} | \
        {(r, 768, 256, False, torch.bfloat16) for r in steps} | {(r, 1000, 256, False, torch.float32) for r in steps}
    assert plan == {k: v for k, v in measured.items() if v is not None}
    for (rows, N, K, gated, out_dtype), how in plan.items():
        assert how in ops._candidates(rows, N, K, gated, out_dtype)
        assert (ops.route_gated(rows, N, K) if gated else ops.route_linear(rows, N, K, out_dtype)) == how
    before = dict(plan)
    calls = []
    monkeypatch.setattr(ops, "_time_ways", lambda runs, *a: calls.append(a) or {how: 1.0 for how in runs})
    plan.clear()
    ops.tune_products(products, max_rows=5)                            # nothing is measured twice
    assert not calls and plan == before
    # a way that is clearly faster replaces the rule's, one that is barely faster does not
    cands = ops._candidates(1, 768, 256, False, torch.bfloat16)
    assert cands == ["library", "skinny", "resident256", "resident512", "sweep"]
    plan.clear()
    assert ops.route_linear(1, 768, 256, torch.bfloat16) == "skinny"            # the rule
    key = (1, 768, 256, False, torch.bfloat16)
    for seconds, choice in (([1.0, 0.95, 0.5, 0.96, 0.97], "resident256"), ([0.9, 0.95, 1.0, 0.96, 0.97], None)):
        monkeypatch.setattr(ops, "_time_ways", lambda runs, *a, seconds=seconds: dict(zip(runs, seconds)))
        plan.clear(); measured.clear()
        ops.tune_products([(ws[0], False, None)], max_rows=1)
        assert plan.get(key) == choice and measured[key] == choice
    other = HipOps(DEV)
    assert other.product_plan == {} and other.route_linear(1, 768, 256, torch.bfloat16) == "skinny"


def test_products_for_the_residual_stream_are_measured_at_some_hundred_rows_too(ops, monkeypatch):
    """Beyond 64 rows only the products whose result goes into the residual stream are measured (the
    library's one product against its batch over pieces of K, each with the norm that takes the result),
    up to the rows a step can bring; other products of that many rows stay with the rule."""
    plan, measured = {}, {}
    monkeypatch.setattr(ops, "product_plan", plan)
    monkeypatch.setattr(ops, "_measured", measured)
    ws = [rnd(160, 2048, dtype=torch.bfloat16, seed=i, scale=0.1) for i in range(2)]
    ops.tune_products([(w, False, "residual") for w in ws] + [(w, False, None) for w in ws], max_rows=2, max_rows_residual=200)
    rows_res = {r for (r, N, K, gated, od) in measured if od == "residual"}
    rows_plain = {r for (r, N, K, gated, od) in measured if od != "residual"}
    assert rows_plain == {1, 2} and rows_res == {1, 2, 96, 128, 192, 256}
    assert ops._rows_step(200, True) == 256 and ops._rows_step(200) == 0 and ops._rows_step(5000, True) == 0
    for (rows, N, K, gated, od), how in plan.items():
        assert how in ops._candidates(rows, N, K, gated, od)
    # what the plan names at 256 rows is what 200 rows get, as shares or as rows; both give the product
    x = rnd(200, 2048, dtype=torch.bfloat16, seed=5)
    want = x.double() @ ws[0].double().t()
    from return_amd.parts.runtime import Slabs
    for how in ("library", "split2", "split8"):
        plan[(256, 160, 2048, False, "residual")] = how
        assert ops.route_linear(200, 160, 2048, "residual") == how
        y = ops.linear_residual(x, ws[0])
        got = y.tensor.double().sum(0) if isinstance(y, Slabs) else y.double()
        assert isinstance(y, Slabs) == how.startswith("split")
        torch.testing.assert_close(got, want, atol=0.3, rtol=2e-2)
    assert ops.route_linear(200, 160, 2048, torch.bfloat16) == "library"


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,N,K", [(65, 331, 120), (128, 128, 32), (129, 257, 264), (300, 1000, 512), (70, 48, 8),
                                   (3000, 4300, 32), (2700, 5130, 64), (5130, 2700, 96), (2570, 5000, 160),
                                   (1290, 10001, 224), (3000, 4500, 256), (4000, 3333, 352), (2048, 6400, 4096)])
def test_tiled_mfma_product(ops, out_dtype, M, N, K):
    """The hand-written tiled products for many rows, edges in every dimension: tiles of 128 x 128 up
    to 128 rows, when K is no multiple of 32 or when larger tiles would be fewer than 160, tiles of 256 x 256
    otherwise, with 1, 2, 3, 5, 7, 8, 11
    and 128 k-steps of 32 (the copies run three stages ahead; the loop's steady part starts at seven)."""
    x = rnd(M, K, dtype=torch.bfloat16, seed=47)
    w = rnd(N, K, dtype=torch.bfloat16, seed=48, scale=0.1)
    ops.own_gemm = True
    try:
        y = ops.linear(x, w, out_dtype=out_dtype)
    finally:
        ops.own_gemm = False
    want = x.double() @ w.double().t()
    assert y.dtype == out_dtype
    if out_dtype == torch.float32:
        torch.testing.assert_close(y.double(), want, atol=1e-4 * K ** 0.5, rtol=1e-5)
    else:
        torch.testing.assert_close(y.double(), want, atol=3e-2, rtol=2e-2)


@pytest.mark.parametrize("M", [1, 2, 3, 8, 9, 16, 17])
@pytest.mark.parametrize("N,K", [(331, 120), (48, 1000), (1000, 4), (70, 4096), (16, 516)])
def test_linear_float32_few_rows(ops, M, N, K):
    """float32 rows times float32 weights: up to 16 rows go to the kernel that streams W once,
    more to the tiled kernel; both are plain 32-bit sums."""
    x = rnd(M, K, seed=91)
    w = rnd(N, K, seed=92, scale=0.3)
    y = ops.linear(x, w)
    assert y.dtype == torch.float32
    torch.testing.assert_close(y.double(), x.double() @ w.double().t(), atol=2e-6 * K ** 0.5 + 1e-6, rtol=1e-5)


@pytest.mark.parametrize("M,own", [(4, False), (40, False), (40, True), (300, False)])
def test_linear_fp32_is_true_fp32(ops, monkeypatch, M, own):
    """Inputs 1 + 2^-12 round to 1 in bf16 and tf32; a true 32-bit product keeps the 2^-11 per term.
    Few rows (the kernel that streams W once), many rows through the library (which the kernel set
    has checked at start to be a 32-bit product) and through the hand-written tiled kernel."""
    assert ops._library_fp32_exact
    monkeypatch.setattr(ops, "own_gemm", own)
    K = 64
    x = torch.full((M, K), 1.0 + 2.0 ** -12, device=DEV)
    w = torch.full((8, K), 1.0 + 2.0 ** -12, device=DEV)
    y = ops.linear(x, w)
    want = K * (1.0 + 2.0 ** -12) ** 2          # 64.03125...
    assert abs(float(y[0, 0]) - want) < 1e-4
    assert abs(float(y[M - 1, 7]) - want) < 1e-4


def _step(q_lens, q_starts, P, pages_of, kv_starts=None):
    """A StepBatch-like object for the attention ops from host lists."""
    n = len(q_lens)
    cu_q = [0]
    for q in q_lens:
        cu_q.append(cu_q[-1] + q)
    cu_p = [0]
    for p in pages_of:
        cu_p.append(cu_p[-1] + len(p))
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    g = types.SimpleNamespace(page_table=i32([p for ps in pages_of for p in ps]), cu_pages=i32(cu_p),
                              kv_start=i32(kv_starts or [0] * n), slot_mapping=None,
                              n_pages=[len(p) for p in pages_of], max_pages=max(len(p) for p in pages_of))
    dec = [i for i, q in enumerate(q_lens) if q == 1]
    pre = [i for i, q in enumerate(q_lens) if q != 1]
    both = bool(dec) and bool(pre)
    extra = dict(n_decode=len(dec), decode_segs=i32(dec) if both else None,
                 max_decode_seq_len=max([q_starts[i] + 1 for i in dec], default=0),
                 n_prefill_tokens=cu_q[-1] - len(dec),
                 prefill_toks=i32([t for i in pre for t in range(cu_q[i], cu_q[i + 1])]) if both else None,
                 prefill_segs=pre)
    from return_amd.engine.batch import prefill_tiles
    extra.update(prefill_tiles={})
    if any(q != 1 for q in q_lens):
        extra.update(prefill_tiles={rows: i32(prefill_tiles(q_lens, q_starts, rows)) for rows in (64, 128)})
    return types.SimpleNamespace(**extra, n_seqs=n, n_tokens=cu_q[-1], cu_q=i32(cu_q), q_start=i32(q_starts),
                                 seq_lens=i32([a + b for a, b in zip(q_starts, q_lens)]), groups=[g],
                                 q_lens=list(q_lens), q_starts=list(q_starts),
                                 all_decode=all(q == 1 for q in q_lens), max_q_len=max(q_lens),
                                 max_seq_len=max(a + b for a, b in zip(q_starts, q_lens)))


ATTN_CASES = [
    # Hq, Hkv, D, P, [(q_len, q_start)], window
    (4, 2, 16, 16, [(5, 0), (17, 0), (33, 0)], 0),
    (6, 1, 32, 32, [(1, 99), (24, 8), (1, 0), (2, 62)], 0),
    (5, 5, 48, 16, [(40, 3), (1, 200)], 0),
    (8, 2, 128, 16, [(1, 500), (1, 17), (1, 0), (1, 255)], 0),
    (8, 2, 128, 64, [(130, 0), (70, 190)], 0),
    (4, 4, 80, 8, [(30, 10), (1, 77)], 12),
    (3, 1, 64, 16, [(64, 64), (1, 128)], 33),
    (2, 1, 256, 16, [(19, 30)], 0),
    (32, 8, 128, 16, [(1, 2047), (1, 63), (1, 64), (1, 65)], 0),
    (16, 1, 64, 32, [(1, 300), (1, 5)], 0),
    (4, 2, 96, 16, [(1, 130), (3, 7), (1, 0)], 0),
    (8, 2, 208, 16, [(1, 150), (1, 1)], 0),
    (6, 2, 32, 8, [(1, 400), (1, 77), (5, 70), (1, 3)], 70),
    (4, 4, 256, 16, [(1, 199)], 0),
    (24, 1, 64, 16, [(1, 100)], 0),
    (40, 2, 128, 16, [(1, 300), (9, 20), (1, 64), (1, 0)], 0),     # 20 heads a kv head: two waves of 16 and 4
    (33, 1, 48, 8, [(1, 77), (1, 200)], 50),
    # head sizes that the MFMA kernels do not take (no multiple of 16, or beyond 256): the plain kernel in both precisions
    (6, 2, 24, 16, [(1, 130), (20, 7), (1, 0), (70, 64)], 0),
    (5, 1, 40, 8, [(1, 300), (33, 0), (1, 17)], 0),
    (4, 4, 72, 16, [(9, 20), (1, 200), (1, 1)], 25),
    (4, 2, 320, 16, [(1, 150), (40, 3), (2, 62)], 0),
    (3, 1, 6, 4, [(1, 99), (17, 0)], 0),
    (2, 1, 512, 16, [(1, 70), (5, 30)], 0),
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("Hq,Hkv,D,P,segs,window", ATTN_CASES)
def test_attention(ops, ref, dtype, Hq, Hkv, D, P, segs, window, monkeypatch):
    monkeypatch.setattr(ops, "prefill_small_tiles", (Hq + D + len(segs)) % 2 == 0)     # tiles of 64 rows in half the cases
    q_lens = [s[0] for s in segs]
    q_starts = [s[1] for s in segs]
    need = [-(-(a + b) // P) for a, b in segs]
    total_pages = sum(need) + 3
    perm = torch.randperm(total_pages, generator=torch.Generator().manual_seed(5)).tolist()
    pages_of = []
    for k in need:
        pages_of.append([perm.pop() for _ in range(k)])
    step = _step(q_lens, q_starts, P, pages_of)
    kp = rnd(total_pages, Hkv, P, D, dtype=dtype, seed=51)
    vp = rnd(total_pages, Hkv, P, D, dtype=dtype, seed=52)
    q = rnd(sum(q_lens), Hq, D, dtype=dtype, seed=53)
    a = torch.zeros_like(q)
    b = torch.zeros_like(q)
    ops.attention(q, a, kp, vp, step, 0, D ** -0.5, window)
    ref.attention(q, b, kp, vp, step, 0, D ** -0.5, window)
    torch.testing.assert_close(a.float(), b.float(), **tol(dtype))


@pytest.mark.parametrize("small_tiles", [False, True])
@pytest.mark.parametrize("key_split", [1, 2])
@pytest.mark.parametrize("D", list(range(16, 257, 16)))
def test_prefill_attention_every_head_size(ops, ref, D, key_split, small_tiles, monkeypatch):
    """The bfloat16 prefill kernel at every head size it takes: whole prompts, portions with
    context, tiles that end inside a page, a window, an odd and an even number of key tiles;
    with one group of waves per q tile and with two that share its keys; with q tiles of 128 rows
    and (up to head size 128, while they are few) of 64."""
    if small_tiles and D > 128:
        pytest.skip("beyond head size 128 the tiles have 64 rows anyway")
    monkeypatch.setattr(ops, "prefill_key_split", key_split)
    monkeypatch.setattr(ops, "prefill_small_tiles", small_tiles)
    for (Hq, Hkv), window in (((4, 2), 0), ((3, 1), 37)):
        P = 16
        segs = [(70, 0), (2, 131), (65, 64), (5, 3), (130, 259), (140, 300)]
        need = [-(-(a + b) // P) for a, b in segs]
        pages_of, nxt = [], 0
        for k in need:
            pages_of.append(list(range(nxt, nxt + k)))
            nxt += k
        step = _step([s[0] for s in segs], [s[1] for s in segs], P, pages_of)
        kp = rnd(nxt, Hkv, P, D, dtype=torch.bfloat16, seed=D)
        vp = rnd(nxt, Hkv, P, D, dtype=torch.bfloat16, seed=D + 1)
        q = rnd(sum(s[0] for s in segs), Hq, D, dtype=torch.bfloat16, seed=D + 2)
        a, b = torch.zeros_like(q), torch.zeros_like(q)
        ops.attention(q, a, kp, vp, step, 0, D ** -0.5, window)
        ref.attention(q, b, kp, vp, step, 0, D ** -0.5, window)
        torch.testing.assert_close(a.float(), b.float(), **tol(torch.bfloat16))


def test_splits_of_the_decode_attention_follow_the_class_the_runner_names(ops):
    """A decode step that names its class (the batch size and context bucket of the graph that serves or would
    serve it) gets the class's splits, whatever its own numbers: the eager step of 12 requests of up to 301 tokens
    and the captured step of 16 rows bound by 512 choose alike, and so sum in the same order. Without a class the
    step's own numbers decide. Few waves: one pass of 64 keys each; the whole-round rule for merging inside the
    workgroup follows the class too."""
    def step(n, longest, rule=None, bound=False):
        return types.SimpleNamespace(n_decode=n, max_decode_seq_len=longest, decode_rule=rule, decode_len_is_bound=bound)
    n_q, n_kv, D = 32, 8, 128
    eager = ops._decode_splits(step(12, 301, rule=(16, 512)), n_q, n_kv, D, 0)
    graph = ops._decode_splits(step(16, 512, rule=(16, 512), bound=True), n_q, n_kv, D, 0)
    assert eager[0] == graph[0] and eager[2] == graph[2] is False
    assert graph[1] == (512 - 1) // graph[0] + 1 and eager[1] == (301 - 1) // eager[0] + 1
    # one request over 2,048 keys: 8 kv heads x 33 chunks are few waves, a pass of 64 keys each
    assert ops._decode_splits(step(1, 2049), n_q, n_kv, D, 0) == (64, 33, False)
    assert ops._decode_splits(step(8, 2049), n_q, n_kv, D, 0)[0] == 128
    # 32 requests x 8 kv heads are one whole round of the CUs (when the chip has 256): merged in the workgroup
    if ops.cu_count == 256:
        assert ops._decode_splits(step(32, 2049), n_q, n_kv, D, 0)[2] is True
        assert ops._decode_splits(step(30, 2049, rule=(32, 4096)), n_q, n_kv, D, 0)[2] is True
        assert ops._decode_splits(step(30, 2049), n_q, n_kv, D, 0)[2] is False


def test_mixed_step_runs_its_two_attention_kernels_side_by_side(ops, ref, monkeypatch):
    """A step of prompt portions beside decoded tokens: the decode kernel and the prefill kernel on two
    streams give the bits they give one after the other, call after call (the second stream is joined
    before anything reads the result), and what the plain reference gives."""
    Hq, Hkv, D, P = 8, 2, 128, 16
    segs = [(1, 700), (300, 40), (1, 5), (1, 1999), (70, 0), (1, 64), (2, 130)]
    need = [-(-(a + b) // P) for a, b in segs]
    perm = torch.randperm(sum(need) + 3, generator=torch.Generator().manual_seed(9)).tolist()
    pages_of = [[perm.pop() for _ in range(k)] for k in need]
    step = _step([s[0] for s in segs], [s[1] for s in segs], P, pages_of)
    assert step.n_decode == 4 and step.n_prefill_tokens == 372
    kp = rnd(sum(need) + 3, Hkv, P, D, dtype=torch.bfloat16, seed=61)
    vp = rnd(sum(need) + 3, Hkv, P, D, dtype=torch.bfloat16, seed=62)
    want = None
    for it in range(6):
        q = rnd(sum(s[0] for s in segs), Hq, D, dtype=torch.bfloat16, seed=70 + it)
        outs = []
        for overlap in (True, False):
            monkeypatch.setattr(ops, "overlap_attention", overlap)
            o = torch.zeros_like(q)
            ops.attention(q, o, kp, vp, step, 0, D ** -0.5, 0)
            outs.append(o * 1)                    # (read on the main stream, right after the call)
        assert torch.equal(outs[0], outs[1]), f"call {it}"
        want = torch.zeros_like(q)
        ref.attention(q, want, kp, vp, step, 0, D ** -0.5, 0)
        torch.testing.assert_close(outs[0].float(), want.float(), **tol(torch.bfloat16))
    assert ops._side_stream is not None


@pytest.mark.parametrize("merge", [0, 2, 4, 8])
@pytest.mark.parametrize("D", list(range(16, 257, 16)))
def test_decode_attention_every_head_size(ops, ref, monkeypatch, D, merge):
    """The bfloat16 decode kernel at every head size it takes, grouped, ungrouped and with more
    query heads to a kv head than one wave takes; with the splits of a request merged by a
    second kernel, and as two, four or eight waves of one workgroup that merges them itself."""
    monkeypatch.setattr(ops, "decode_merge_round", 1 if merge else 0)
    monkeypatch.setattr(ops, "decode_merge_waves", merge)
    for Hq, Hkv in ((4, 1), (3, 3), (16, 2), (34, 2)):
        P = 16
        segs = [(1, 150), (1, 1), (1, 64), (1, 700)]
        need = [-(-(a + b) // P) for b, a in segs]
        pages_of, nxt = [], 0
        for k in need:
            pages_of.append(list(range(nxt, nxt + k)))
            nxt += k
        step = _step([1] * len(segs), [s[1] for s in segs], P, pages_of)
        kp = rnd(nxt, Hkv, P, D, dtype=torch.bfloat16, seed=D)
        vp = rnd(nxt, Hkv, P, D, dtype=torch.bfloat16, seed=D + 1)
        q = rnd(len(segs), Hq, D, dtype=torch.bfloat16, seed=D + 2)
        a, b = torch.zeros_like(q), torch.zeros_like(q)
        ops.attention(q, a, kp, vp, step, 0, D ** -0.5, 0)
        ref.attention(q, b, kp, vp, step, 0, D ** -0.5, 0)
        torch.testing.assert_close(a.float(), b.float(), **tol(torch.bfloat16))
        S, W, merged = ops._decode_splits(step, Hq, Hkv, D, 0)
        assert merged == bool(merge) and (not merge or W == min(merge, ops.lib.ra_attention_decode_merge_waves(D)))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("q_len", [1, 2, 7, 70])
@pytest.mark.parametrize("older_wins", [True, False])
def test_attention_edges_of_window_and_causality(ops, dtype, q_len, older_wins):
    """Keys are made so that one edge of what a query may see decides its output. older_wins: the
    score grows with the key's age, so every query row picks the oldest key of its window and a
    window that is one key too long or too short shows; else it grows with the position, every row
    picks itself, and a row that sees the key after it shows. The edges of the rows straddle page
    borders, the pages lie scattered; one token goes to the decode kernel, more to the prefill kernel."""
    Hq, Hkv, D, P, window = 4, 2, 64, 16, 37
    start = 220 - q_len                                  # the last row sits at position 219
    L = start + q_len
    n_pages = -(-L // P)
    perm = torch.randperm(n_pages + 5, generator=torch.Generator().manual_seed(9)).tolist()
    pages = perm[:n_pages]
    step = _step([q_len], [start], P, [pages])
    pos = torch.arange(L)
    mag = (256 - pos if older_wins else pos + 1).float()         # whole numbers up to 256: exact in bfloat16
    k = torch.zeros(L, Hkv, D)
    k[:, :, 0] = mag[:, None]
    v = rnd(L, Hkv, D, seed=71).cpu()
    kp = torch.zeros(n_pages + 5, Hkv, P, D)
    vp = torch.zeros_like(kp)
    for i in range(L):
        kp[pages[i // P], :, i % P] = k[i]               # pools are [pages, kv heads, rows in a page, D]
        vp[pages[i // P], :, i % P] = v[i]
    kp, vp = kp.to(dtype).to(DEV), vp.to(dtype).to(DEV)
    q = torch.zeros(q_len, Hq, D)
    q[:, :, 0] = 96.0                                    # 96 * 1 / sqrt(64) = 12 per step of the magnitude
    q = q.to(dtype).to(DEV)
    out = torch.zeros_like(q)
    ops.attention(q, out, kp, vp, step, 0, D ** -0.5, window)
    for r in range(q_len):
        pos_q = start + r
        pick = max(0, pos_q - window + 1) if older_wins else pos_q
        want = v[pick].to(dtype).float().repeat_interleave(Hq // Hkv, dim=0)      # [Hq, D]
        torch.testing.assert_close(out[r].float().cpu(), want, atol=2e-2 if dtype == torch.bfloat16 else 1e-4,
                                   rtol=0, msg=lambda m: f"row {r} (position {pos_q}) should have picked key {pick}: {m}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_far_key_stands_out(ops, dtype):
    """One key far back among hundreds is made to dominate: the output must be its value."""
    Hq, Hkv, D, P, L = 4, 2, 64, 16, 700
    pages = list(range(-(-L // P)))
    step = _step([1], [L - 1], P, [pages])
    kp = rnd(len(pages), Hkv, P, D, dtype=dtype, seed=61, scale=0.1)
    vp = rnd(len(pages), Hkv, P, D, dtype=dtype, seed=62)
    q = rnd(1, Hq, D, dtype=dtype, seed=63, scale=0.1)
    far = 37
    kp[far // P, :, far % P] = (q.view(Hq, D)[::2] * 400).to(dtype)      # kv head h gets query head 2h, scaled up
    out = torch.zeros_like(q)
    ops.attention(q, out, kp, vp, step, 0, 1.0, 0)
    want = vp[far // P, :, far % P].float()
    torch.testing.assert_close(out[0, ::2].float(), want, atol=3e-2, rtol=3e-2)


@pytest.mark.parametrize("split", [0, 64, 192, "merge", "merge8"])
@pytest.mark.parametrize("D,Hq,Hkv,normed,rotated,window", [
    (128, 8, 2, True, True, 0), (64, 4, 4, True, True, 0), (192, 3, 1, False, True, 0), (256, 4, 2, True, False, 0),
    (128, 40, 2, True, True, 0), (64, 6, 2, True, True, 70), (128, 4, 1, False, False, 0)])
def test_decode_attention_that_prepares_q_k_v_itself(ops, monkeypatch, D, Hq, Hkv, normed, rotated, window, split):
    """The decode kernel fed with the projection's output (it norms and rotates q and k and writes
    k and v into the cache) against the preparation kernel followed by the decode kernel: new
    tokens at the first place, at the edges of pages, passes and splits, and far out."""
    merge = str(split).startswith("merge")
    monkeypatch.setattr(ops, "decode_split_tokens", 0 if merge else split)
    monkeypatch.setattr(ops, "decode_merge_round", 1 if merge else 0)
    monkeypatch.setattr(ops, "decode_merge_waves", 8 if split == "merge8" else 0)
    P = 16
    starts = [0, 1, 15, 16, 63, 64, 65, 127, 128, 191, 192, 700]
    need = [-(-(a + 1) // P) for a in starts]
    perm = torch.randperm(sum(need) + 3, generator=torch.Generator().manual_seed(D)).tolist()
    pages_of = [[perm.pop() for _ in range(k)] for k in need]
    step = _step([1] * len(starts), starts, P, pages_of)
    n = len(starts)
    kp = rnd(sum(need) + 3, Hkv, P, D, dtype=torch.bfloat16, seed=1)
    vp = rnd(sum(need) + 3, Hkv, P, D, dtype=torch.bfloat16, seed=2)
    qkv = rnd(n, (Hq + 2 * Hkv) * D, dtype=torch.bfloat16, seed=3)
    wq = (1 + 0.1 * rnd(D, seed=4)) if normed else None
    wk = (1 + 0.1 * rnd(D, seed=5)) if normed else None
    pos = torch.arange(1024, device=DEV)[:, None] * (1.0 / 10000 ** (torch.arange(D // 2, device=DEV) / (D // 2)))[None]
    cos, sin = (pos.cos().contiguous(), pos.sin().contiguous()) if rotated else (None, None)
    R = D if rotated else 0
    positions = torch.tensor(starts, dtype=torch.int32, device=DEV)
    slots = torch.tensor([pages_of[i][a // P] * P + a % P for i, a in enumerate(starts)], dtype=torch.int32, device=DEV)
    # two kernels
    k1, v1 = kp.clone(), vp.clone()
    q = torch.zeros(n, Hq, D, dtype=torch.bfloat16, device=DEV)
    ops.qkv_prepare(qkv, Hq, Hkv, D, wq, wk, 1e-5, positions, cos, sin, R, q, k1, v1, slots)
    want = torch.zeros_like(q)
    ops.attention(q, want, k1, v1, step, 0, D ** -0.5, window)
    # one kernel
    k2, v2 = kp.clone(), vp.clone()
    got = torch.zeros_like(q)
    assert ops.attention_qkv(qkv, got, k2, v2, step, 0, D ** -0.5, window, Hq, Hkv, D, wq, wk, 1e-5, cos, sin, R)
    assert torch.equal(v1, v2)                                         # values are copied
    torch.testing.assert_close(k2.float(), k1.float(), atol=0, rtol=2 ** -7)      # keys: the last bit of the rounding at most
    assert (k2 != k1).float().mean().item() < 1e-3
    torch.testing.assert_close(got.float(), want.float(), **tol(torch.bfloat16))
    # a step with a portion in it is not taken
    mixed = _step([1, 3], [5, 0], P, [[0], [1]])
    assert not ops.attention_qkv(qkv[:4], got[:4], k2, v2, mixed, 0, 1.0, 0, Hq, Hkv, D, wq, wk, 1e-5, cos, sin, R)


@pytest.mark.parametrize("split", [0, 64, 256, 1024])
@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_over_a_long_context(ops, ref, monkeypatch, dtype, split):
    """40,000 keys in scattered pages: a decoded token at the end of them, one after five keys, and
    a portion of 300 query rows whose first row sees 39,700 keys; in one step. With splits of the
    decode kernel's own choice and of 64, 256 and 1,024 keys (625, 157 and 40 splits, which the merge
    takes in eight, eight and four groups of threads)."""
    monkeypatch.setattr(ops, "decode_split_tokens", split)
    Hq, Hkv, D, P = 8, 2, 128, 16
    segs = [(1, 39_999), (1, 5), (300, 39_700)]
    need = [-(-(a + b) // P) for a, b in segs]
    perm = torch.randperm(sum(need) + 7, generator=torch.Generator().manual_seed(3)).tolist()
    pages_of = [[perm.pop() for _ in range(k)] for k in need]
    step = _step([s[0] for s in segs], [s[1] for s in segs], P, pages_of)
    kp = rnd(sum(need) + 7, Hkv, P, D, dtype=dtype, seed=81)
    vp = rnd(sum(need) + 7, Hkv, P, D, dtype=dtype, seed=82)
    q = rnd(sum(s[0] for s in segs), Hq, D, dtype=dtype, seed=83)
    a, b = torch.zeros_like(q), torch.zeros_like(q)
    ops.attention(q, a, kp, vp, step, 0, D ** -0.5, 0)
    ref.attention(q, b, kp, vp, step, 0, D ** -0.5, 0)
    torch.testing.assert_close(a.float(), b.float(), **tol(dtype))


@pytest.mark.parametrize("V", [331, 5000])
def test_sample_greedy_and_logprob(ops, V):
    logits = rnd(6, V, seed=71, scale=3.0)
    z = torch.zeros(6, device=DEV)
    out = ops.sample(logits, z, torch.zeros(6, dtype=torch.int32, device=DEV), torch.ones(6, device=DEV), z)
    tok = out[:, 0].long()
    assert torch.equal(tok, logits.argmax(-1))
    lp = out[:, 1].contiguous().view(torch.float32)
    want = logits.double().log_softmax(-1).gather(1, tok[:, None])[:, 0]
    torch.testing.assert_close(lp.double(), want, atol=1e-4, rtol=1e-5)


@pytest.mark.parametrize("V", [97, 1000, 20001])
def test_sample_matches_plain_draw(ops, ref, V):
    M = 64
    logits = rnd(M, V, seed=72, scale=2.0)
    g = torch.Generator().manual_seed(9)
    u = torch.rand(M, generator=g).to(DEV)
    temp = torch.tensor([0.7, 1.0, 1.3, 0.0] * (M // 4), device=DEV)
    top_k = torch.tensor([0, 5, 0, 3, 50, 0, 1, 0] * (M // 8), dtype=torch.int32, device=DEV)
    top_p = torch.tensor([1.0, 1.0, 0.9, 0.5, 0.3, 0.0, 1.0, 0.95] * (M // 8), device=DEV)
    path = torch.full((M,), -1, dtype=torch.int32, device=DEV)
    a = ops.sample(logits, temp, top_k, top_p, u, path=path)
    b = ref.sample(logits, temp, top_k, top_p, u)
    same = (a[:, 0] == b[:, 0]).float().mean().item()
    assert same == 1.0, (a[:, 0].tolist(), b[:, 0].tolist())
    # a small vocabulary fits the list of the largest logits: every row that needs a threshold takes it from
    # there; 20,001 flat logits (an odd number: no 16-byte loads) do not fit, and the search goes over the row
    needs = (temp > 0) & ((top_k > 0) | (top_p < 1))
    assert torch.equal(path[needs], torch.full_like(path[needs], 1 if V <= 8192 else 2))
    assert int(path[~needs].abs().sum()) == 0
    torch.testing.assert_close(a[:, 1].contiguous().view(torch.float32), b[:, 1].contiguous().view(torch.float32),
                               atol=1e-4, rtol=1e-5)


def test_sample_at_the_full_vocabulary(ops):
    """top-k and top-p at a vocabulary of 151,936 (the threshold search over the whole row, pass by
    pass): every row's token is where the plain distribution's running sum, in vocabulary order,
    passes the row's uniform number; peaked and flat rows, ties above the boundary, k = 1, p near 0."""
    from tests.plain import qwen3_plain as plain
    V, M = 151936, 32
    logits = rnd(M, V, seed=73, scale=3.0)
    logits[1] = (logits[1] * 0.05)                                # flat: top-p keeps tens of thousands
    logits[2, 1000:1040] = logits[2].max() + 1.0                  # forty tokens tie at the top
    logits[3, 5000:5003] = logits[3].max()                        # three more tokens tie with the largest (all above the boundary)
    g = torch.Generator().manual_seed(11)
    u = torch.rand(M, generator=g).to(DEV)
    temp = torch.tensor([0.7, 1.0, 1.3, 0.9] * (M // 4), device=DEV)
    top_k = torch.tensor([0, 0, 50, 0, 20, 1, 0, 3000] * (M // 8), dtype=torch.int32, device=DEV)
    top_p = torch.tensor([0.9, 0.95, 1.0, 0.5, 0.8, 1.0, 0.01, 0.99] * (M // 8), device=DEV)
    out = ops.sample(logits, temp, top_k, top_p, u).cpu()
    for r in range(M):
        d = plain.sample_distribution(logits[r].cpu(), float(temp[r]), int(top_k[r]), float(top_p[r]))
        tok = int(out[r, 0])
        assert d[tok] > 0, f"row {r}: token {tok} is not among the kept ones"
        c = d.cumsum(0)
        before = float(c[tok - 1]) if tok else 0.0
        assert before - 1e-4 <= float(u[r]) <= float(c[tok]) + 1e-4, (r, tok, before, float(u[r]), float(c[tok]))
        lp = out[r, 1:2].contiguous().view(torch.float32)
        assert abs(float(lp) - plain.chosen_logprob(logits[r].cpu(), tok)) < 1e-3


@pytest.mark.parametrize("V,path", [(1000, 1), (20001, 2), (151936, 2)])
def test_sample_cuts_ties_at_a_boundary_in_vocabulary_order(ops, ref, V, path):
    """Logits from a handful of values, so that hundreds of tokens tie at every boundary: exactly top_k
    tokens stay (rollout/model.py:45-50 keeps topk(k)), of the tying ones the first in the vocabulary, as the
    plain rule's stable sort has them; of the tokens that tie at the top-p boundary those before which at most
    top_p of the mass lies (the crossing token stays, rollout/model.py:51-55). Every row's token is the plain
    draw's, from the list of the largest logits (a vocabulary that fits it) and from the whole row."""
    M = 64
    g = torch.Generator().manual_seed(V)
    logits = torch.randint(0, 5, (M, V), generator=g).float()
    logits[:, 7] = 5.0                                            # one largest, so that the rows are not flat at the top
    logits = logits.to(DEV)
    u = torch.rand(M, generator=g).to(DEV)
    temp = torch.tensor([1.0, 0.7, 1.5, 1.0] * (M // 4), device=DEV)
    top_k = torch.tensor([50, 0, 333, 2, 0, 1000, 7, 0] * (M // 8), dtype=torch.int32, device=DEV)
    top_p = torch.tensor([1.0, 0.3, 0.9, 1.0, 0.05, 0.5, 0.6, 0.999] * (M // 8), device=DEV)
    way = torch.full((M,), -1, dtype=torch.int32, device=DEV)
    a = ops.sample(logits, temp, top_k, top_p, u, path=way)
    b = ref.sample(logits, temp, top_k, top_p, u)
    assert a[:, 0].tolist() == b[:, 0].tolist()
    assert set(way.tolist()) == {path}
    # and the kept set itself, row by row: a sweep of uniform numbers draws exactly the plain rule's tokens
    from tests.plain import qwen3_plain as plain
    for r in (0, 1, 3, 6):
        d = plain.sample_distribution(logits[r].cpu(), float(temp[r]), int(top_k[r]), float(top_p[r]))
        support = set(d.nonzero().flatten().tolist())
        n = 2048
        sweep = ((torch.arange(n) + 0.5) / n).to(DEV)
        rows = logits[r:r + 1].expand(n, V).contiguous()
        out = ops.sample(rows, temp[r:r + 1].expand(n).contiguous(), top_k[r:r + 1].expand(n).contiguous(),
                         top_p[r:r + 1].expand(n).contiguous(), sweep)
        drawn = set(out[:, 0].tolist())
        assert drawn <= support, f"row {r}: tokens outside the kept set were drawn: {sorted(drawn - support)[:5]}"
        if len(support) <= 64:
            assert drawn == support, f"row {r}: kept tokens that no uniform number reaches: {sorted(support - drawn)[:5]}"
        if int(top_k[r]) > 0 and float(top_p[r]) >= 1.0:
            assert len(support) == int(top_k[r])


def test_sample_from_the_list_of_the_largest_logits_and_from_the_whole_row(ops):
    """Rows shaped like a language model's (a bulk of 151,936 logits far below a few hundred large ones)
    take their thresholds and their token from the list of the largest; rows whose large ones crowd into
    one wave's run of the row, whose k is more than the list holds, or whose top_p reaches into the bulk
    go over the whole row. Either way the token is where the plain distribution's running sum, in
    vocabulary order, passes the row's uniform number."""
    from tests.plain import qwen3_plain as plain
    V = 151936
    g = torch.Generator().manual_seed(21)
    base = torch.randn(V, generator=g) * 1.5
    def row(n_large, where, top=12.0):
        x = base.clone()
        idx = where[torch.randperm(len(where), generator=g)[:n_large]]
        x[idx] = 14.0 + 8.0 * torch.rand(n_large, generator=g)          # the large ones: 14 to 22
        x[idx[0]] = 14.0 + top                                           # and the largest
        return x
    everywhere, crowded = torch.arange(V), torch.arange(3000, 9000)
    cases = [   # logits, temperature, top_k, top_p, path expected
        (row(300, everywhere), 1.0, 0, 0.9, 1), (row(300, everywhere), 1.0, 40, 1.0, 1),
        (row(300, everywhere), 0.7, 100, 0.8, 1), (row(2000, everywhere), 1.2, 0, 0.95, 1),
        (row(2000, everywhere), 1.0, 1500, 0.99, 1), (row(300, everywhere), 1.0, 1, 1.0, 1),
        (row(300, everywhere), 1.0, 0, 0.01, 1), (row(40, everywhere), 1.0, 0, 0.999, 1),
        (row(700, crowded), 1.0, 0, 0.9, 2),                 # more than 512 large ones in one wave's run
        (row(300, everywhere), 1.0, 5000, 1.0, 2),           # k beyond the list
        (row(1, everywhere, top=9.0), 1.0, 0, 0.999999, 2),  # the list (one token) has less than top_p of the mass: the boundary lies in the bulk
        (row(3, everywhere, top=3.0), 4.0, 0, 0.9, 2),       # a hot row: the whole vocabulary is within the span
        (row(300, everywhere), 1.0, 0, 1.0, 0),              # no threshold at all
    ]
    M = len(cases)
    logits = torch.stack([c[0] for c in cases]).to(DEV)
    temp = torch.tensor([c[1] for c in cases], device=DEV)
    top_k = torch.tensor([c[2] for c in cases], dtype=torch.int32, device=DEV)
    top_p = torch.tensor([c[3] for c in cases], device=DEV)
    for seed in (1, 2, 3):
        u = torch.rand(M, generator=torch.Generator().manual_seed(seed)).to(DEV)
        path = torch.full((M,), -1, dtype=torch.int32, device=DEV)
        out = ops.sample(logits, temp, top_k, top_p, u, path=path).cpu()
        assert path.tolist() == [c[4] for c in cases]
        for r in range(M):
            d = plain.sample_distribution(logits[r].cpu(), float(temp[r]), int(top_k[r]), float(top_p[r]))
            tok = int(out[r, 0])
            assert d[tok] > 0, f"row {r}: token {tok} is not among the kept ones"
            c = d.cumsum(0)
            before = float(c[tok - 1]) if tok else 0.0
            assert before - 1e-4 <= float(u[r]) <= float(c[tok]) + 1e-4, (r, tok, before, float(u[r]), float(c[tok]))
            lp = out[r, 1:2].contiguous().view(torch.float32)
            assert abs(float(lp) - plain.chosen_logprob(logits[r].cpu(), tok)) < 1e-3


def test_sample_distribution(ops):
    """Plain temperature sampling draws from softmax(logits / T): chi-square on a tiny vocabulary."""
    V, N = 7, 20000
    logits = torch.tensor([[0.0, 1.0, 2.0, -1.0, 0.5, 1.5, -2.0]], device=DEV).repeat(N, 1)
    u = torch.rand(N, generator=torch.Generator().manual_seed(1)).to(DEV)
    temp = torch.full((N,), 0.8, device=DEV)
    out = ops.sample(logits, temp, torch.zeros(N, dtype=torch.int32, device=DEV), torch.ones(N, device=DEV), u)
    counts = torch.bincount(out[:, 0].long().cpu(), minlength=V).double()
    p = (logits[0].double().cpu() / 0.8).softmax(-1)
    chi2 = float(((counts - N * p) ** 2 / (N * p)).sum())
    assert chi2 < 30.0, (chi2, counts.tolist())


@pytest.mark.parametrize("V", [50, 20001])
@pytest.mark.parametrize("fill", [float("-inf"), float("nan")])
def test_sample_of_a_row_without_a_largest_value(ops, V, fill):
    """A row that is all -inf (or all NaN, as after an overflow upstream) has no largest value: every
    way of choosing gives token 0 and a logprob that is no number, reads nothing beyond the row, and
    leaves the rows beside it alone."""
    M = 8
    logits = rnd(M, V, seed=74, scale=2.0)
    logits[1::2] = fill
    temp = torch.tensor([0.0, 0.0, 1.0, 1.0, 0.8, 0.8, 1.2, 1.2], device=DEV)
    top_k = torch.tensor([0, 0, 0, 0, 5, 5, 0, 0], dtype=torch.int32, device=DEV)
    top_p = torch.tensor([1.0, 1.0, 1.0, 1.0, 1.0, 1.0, 0.9, 0.9], device=DEV)
    u = torch.full((M,), 0.5, device=DEV)
    out = ops.sample(logits, temp, top_k, top_p, u).cpu()
    torch.cuda.synchronize()
    lp = out[:, 1].contiguous().view(torch.float32)
    assert out[1::2, 0].tolist() == [0, 0, 0, 0]
    assert not torch.isfinite(lp[1::2]).any()
    assert torch.isfinite(lp[0::2]).all() and ((out[0::2, 0] >= 0) & (out[0::2, 0] < V)).all()
    assert int(out[0, 0]) == int(logits[0].argmax())


def test_calls_that_do_not_fit_are_refused_before_anything_runs(ops):
    """Shapes, dtypes, devices and layouts that a kernel does not take raise KernelError on the
    host; sizes beyond a kernel's limits too."""
    from return_amd.kernels.hip_ops import KernelError
    bf, f32 = torch.bfloat16, torch.float32
    x, w = rnd(4, 64, dtype=bf), rnd(8, 64, dtype=bf)
    bad = [
        ("weight of another width", lambda: ops.linear(x, rnd(8, 48, dtype=bf))),
        ("weight of another dtype", lambda: ops.linear(x, rnd(8, 64))),
        ("x on the host", lambda: ops.linear(x.cpu(), w)),
        ("x not contiguous", lambda: ops.linear(rnd(64, 4, dtype=bf).t(), w)),
        ("gate-up with an odd number of rows", lambda: ops.linear_silu_mul(x, rnd(9, 64, dtype=bf))),
        ("embedding into bf16", lambda: ops.embed(rnd(10, 64, dtype=bf), torch.zeros(4, dtype=torch.int32, device=DEV),
                                                  torch.zeros(4, 64, dtype=bf, device=DEV))),
        ("ids as int64", lambda: ops.embed(rnd(10, 64, dtype=bf), torch.zeros(4, dtype=torch.int64, device=DEV),
                                           torch.zeros(4, 64, device=DEV))),
        ("norm weight of another size", lambda: ops.add_rmsnorm(rnd(4, 64), None, rnd(48), 1e-6, rnd(4, 64, dtype=bf))),
        ("delta of another shape", lambda: ops.add_rmsnorm(rnd(4, 64), rnd(3, 64, dtype=bf), rnd(64), 1e-6,
                                                           rnd(4, 64, dtype=bf))),
        ("silu-mul widths", lambda: ops.silu_mul(rnd(4, 100, dtype=bf), rnd(4, 60, dtype=bf))),
        ("sampling options of another length", lambda: ops.sample(
            rnd(3, 50), torch.zeros(2, device=DEV), torch.zeros(3, dtype=torch.int32, device=DEV),
            torch.ones(3, device=DEV), torch.zeros(3, device=DEV))),
        ("logits in bf16", lambda: ops.sample(
            rnd(3, 50, dtype=bf), torch.zeros(3, device=DEV), torch.zeros(3, dtype=torch.int32, device=DEV),
            torch.ones(3, device=DEV), torch.zeros(3, device=DEV))),
    ]
    # attention: heads that do not divide, a head size beyond the plain kernel's, pools that do not fit
    step = _step([1], [5], 16, [[0]])
    for Hq, Hkv, D, why in ((3, 2, 16, "heads"), (2, 2, 528, "head size")):
        q = rnd(1, Hq, D, dtype=bf)
        kp = rnd(1, Hkv, 16, D, dtype=bf)
        bad.append((f"attention: {why}", lambda q=q, kp=kp: ops.attention(q, torch.zeros_like(q), kp, kp.clone(), step, 0, 1.0, 0)))
    q = rnd(1, 4, 32, dtype=bf)
    bad.append(("attention: pool of another head size",
                lambda: ops.attention(q, torch.zeros_like(q), rnd(1, 2, 16, 16, dtype=bf), rnd(1, 2, 16, 16, dtype=bf), step, 0, 1.0, 0)))
    bad.append(("attention: output of another shape",
                lambda: ops.attention(q, torch.zeros(2, 4, 32, dtype=bf, device=DEV), rnd(1, 2, 16, 32, dtype=bf),
                                      rnd(1, 2, 16, 32, dtype=bf), step, 0, 1.0, 0)))
    for name, call in bad:
        with pytest.raises(KernelError):
            call()
            pytest.fail(f"{name}: was not refused")
    torch.cuda.synchronize()
