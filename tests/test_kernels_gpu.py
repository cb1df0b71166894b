"""Each HIP kernel alone against the plain formulas, at sizes other than the
tiny models' (odd widths, several head sizes, page sizes 4/8/16, windows)."""
import math

import pytest
import torch

from plain import llama_plain as P

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


def tol(dtype, f32=2e-5, bf16=2e-2):
    return dict(rtol=f32, atol=f32) if dtype == torch.float32 else dict(rtol=bf16, atol=bf16)


@pytest.fixture(scope="module")
def ops():
    from lyapunov_engine_amd.kernels import ops as o
    o.require_gpu()
    return o


def rnd(*shape, dtype=torch.float32, scale=1.0, seed=0):
    g = torch.Generator().manual_seed(seed + sum(shape))
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


# ------------------------------------------------------------------- embedding
@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding(ops, dtype):
    V, H, T = 1000, 192, 37
    table = rnd(V, H, dtype=dtype)
    ids = torch.randint(0, V, (T,), generator=torch.Generator().manual_seed(1), dtype=torch.int32)
    out = torch.empty(T, H, dtype=torch.float32, device=DEV)
    ops.embedding(ids.to(DEV), table.to(DEV), out)
    torch.testing.assert_close(out.cpu(), table.float()[ids.long()], rtol=0, atol=0)


# --------------------------------------------------------------------- rmsnorm
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,T", [(96, 1), (1000, 7), (2048, 33), (4100, 3)])
def test_rmsnorm(ops, dtype, H, T):
    eps = 1e-5
    h = rnd(T, H, seed=3)
    w = (1 + 0.1 * rnd(H, seed=4)).to(dtype)
    out = torch.empty(T, H, dtype=dtype, device=DEV)
    hd = h.to(DEV)
    ops.rmsnorm(hd, w.to(DEV), eps, out)
    want = P.rms_norm(h.double(), w.double(), eps)
    torch.testing.assert_close(out.cpu().double(), want, **tol(dtype, 1e-5, 1e-2))
    torch.testing.assert_close(hd.cpu(), h, rtol=0, atol=0)  # no delta: the stream is untouched


@pytest.mark.parametrize("dtype", DTYPES)
def test_rmsnorm_adds_the_residual_in_32_bit(ops, dtype):
    T, H, eps = 9, 200, 1e-6
    h, delta = rnd(T, H, seed=5), rnd(T, H, seed=6, dtype=dtype)
    w = rnd(H, seed=7).to(dtype)
    hd = h.to(DEV)
    out = torch.empty(T, H, dtype=dtype, device=DEV)
    ops.rmsnorm(hd, w.to(DEV), eps, out, delta=delta.to(DEV))
    total = h + delta.float()
    torch.testing.assert_close(hd.cpu(), total, rtol=0, atol=0)  # the sum lands in the float stream, unrounded
    torch.testing.assert_close(out.cpu().double(), P.rms_norm(total.double(), w.double(), eps), **tol(dtype, 1e-5, 1e-2))
    # rows: only the picked rows are normed and the stream is left alone
    rows = torch.tensor([8, 0, 3], dtype=torch.int32)
    hd2 = h.to(DEV)
    out2 = torch.empty(3, H, dtype=dtype, device=DEV)
    ops.rmsnorm(hd2, w.to(DEV), eps, out2, delta=delta.to(DEV), rows=rows.to(DEV))
    torch.testing.assert_close(hd2.cpu(), h, rtol=0, atol=0)
    torch.testing.assert_close(out2.cpu().double(), P.rms_norm(total.double(), w.double(), eps)[rows.long()],
                               **tol(dtype, 1e-5, 1e-2))


# ---------------------------------------------------------------------- swiglu
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("I,T", [(172, 5), (512, 1), (8192, 3)])
def test_swiglu(ops, dtype, I, T):
    gu = rnd(T, 2 * I, dtype=dtype, scale=2.0, seed=8)
    out = torch.empty(T, I, dtype=dtype, device=DEV)
    ops.swiglu(gu.to(DEV), out)
    torch.testing.assert_close(out.cpu().double(), P.swiglu(gu.double()), **tol(dtype, 1e-5, 1e-2))


@pytest.mark.parametrize("dtype", DTYPES)
def test_swiglu_in_tiles_and_inside_the_product(ops, dtype):
    """Gates and ups in tiles of 16 columns, and the few-rows product that gates
    in its epilogue, against the plain gate-first formula."""
    I, K = 48, 128
    g = torch.Generator().manual_seed(2)
    wg, wu = (torch.randn(I, K, generator=g) * 0.1).to(dtype), (torch.randn(I, K, generator=g) * 0.1).to(dtype)
    w = torch.stack([wg.view(-1, 8, K), wu.view(-1, 8, K)], dim=1).reshape(2 * I, K).contiguous()
    for M in (1, 7, 33, 64, 70):
        x = (torch.randn(M, K, generator=g)).to(dtype)
        want = P.mlp(x.double(), wg.double(), wu.double(), torch.eye(I, dtype=torch.float64))
        got = ops.linear_swiglu(x.to(DEV), w.to(DEV), 8)
        torch.testing.assert_close(got.cpu().double(), want, **tol(dtype, 1e-5, 2e-2))
    gu = rnd(5, 2 * I, dtype=dtype, seed=3)
    out = torch.empty(5, I, dtype=dtype, device=DEV)
    ops.swiglu(gu.to(DEV), out, 8)
    tiles = gu.double().view(5, -1, 2, 8)
    want = torch.nn.functional.silu(tiles[:, :, 0]) * tiles[:, :, 1]
    torch.testing.assert_close(out.cpu().double(), want.reshape(5, I), **tol(dtype, 1e-5, 1e-2))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,N,K", [(1, 2048, 2048), (8, 2048, 8192), (33, 96, 1024), (64, 515, 4096), (5, 4096, 2048)])
def test_linear_partial_sums(ops, dtype, M, N, K):
    """A product that comes back in slices of the inner dimension: the slices add
    up to the product, through sum_parts and through the norm's residual add."""
    a, w = rnd(M, K, dtype=dtype, seed=21), rnd(N, K, dtype=dtype, scale=0.05, seed=22)
    want = a.double() @ w.double().T
    bound = a.double().abs() @ w.double().abs().T
    y = ops.linear(a.to(DEV), w.to(DEV), may_split=True)
    rel = 2e-6 if dtype == torch.float32 else 1e-5
    if y.dim() == 3:
        assert y.dtype == torch.float32 and y.shape[1:] == (M, N) and y.shape[0] > 1
        assert ((y.cpu().double().sum(0) - want).abs() <= rel * bound + 1e-30).all()
        total = ops.sum_parts(y, torch.float32)
        assert ((total.cpu().double() - want).abs() <= rel * bound + 1e-30).all()
        h = rnd(M, N, seed=23).to(DEV)
        h0 = h.clone()
        out = torch.empty(M, N, dtype=dtype, device=DEV)
        ops.rmsnorm(h, torch.ones(N, dtype=dtype, device=DEV), 1e-5, out, delta=y)
        assert (((h - h0).cpu().double() - want).abs() <= rel * bound + 1e-5).all()
        torch.testing.assert_close(out.cpu().double(), P.rms_norm(h.cpu().double(), torch.ones(N, dtype=torch.float64), 1e-5),
                                   **tol(dtype, 1e-5, 1e-2))
    else:
        assert N >= 4096 or K < 1024  # only products with few output features and a long inner dimension are sliced
        assert ((y.cpu().double() - want).abs() <= (1e-2 if dtype == torch.bfloat16 else rel) * bound + 1e-30).all()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,N,K", [(1, 2048, 2048), (8, 2048, 8192), (8, 100, 192), (5, 515, 1024), (8, 4096, 1024),
                                   (3, 4101, 384), (7, 3072, 256),
                                   # 9 to 16 rows: two blocks of 8 tokens over one set of weights
                                   (9, 2048, 8192), (16, 2048, 2048), (12, 515, 1024), (13, 4101, 384), (16, 100, 192)])
def test_product_added_to_the_residual_stream_in_its_own_kernel(ops, dtype, M, N, K):
    """A projection of few rows handed on instead of run (pending=True) and
    then added to the float residual stream by the product kernel itself."""
    a, w = rnd(M, K, dtype=dtype, seed=31), rnd(N, K, dtype=dtype, scale=0.05, seed=32)
    want = a.double() @ w.double().T
    bound = a.double().abs() @ w.double().abs().T
    p = ops.linear(a.to(DEV), w.to(DEV), may_split=True, pending=True)
    assert isinstance(p, ops.PendingLinear)
    h0 = rnd(M, N, seed=33)
    h = h0.to(DEV)
    assert ops.linear_residual(h, p) is True
    rel = 2e-6 if dtype == torch.float32 else 1e-5
    assert (((h.cpu() - h0).double() - want).abs() <= rel * bound + 2e-6 * h0.abs() + 1e-6).all()
    # whoever cannot fold it in runs it: the same product (rounded to bfloat16 unless it comes in slices)
    loose = 1e-2 if dtype == torch.bfloat16 and p.run().dim() == 2 else rel
    assert ((ops.as_delta(p, torch.float32).cpu().double() - want).abs() <= loose * bound + 1e-30).all()
    # with more rows the product is not handed on
    big = ops.linear(rnd(ops.PENDING_MAX_ROWS + 1, K, dtype=dtype).to(DEV), w.to(DEV), may_split=True, pending=True)
    assert isinstance(big, torch.Tensor)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,K,J", [(1, 2048, 192), (8, 192, 192), (5, 1024, 256), (7, 256, 384), (8, 320, 128), (6, 4096, 256),
                                   (9, 2048, 256), (16, 1024, 384), (11, 320, 192), (16, 4096, 128)])
def test_norm_folded_into_the_products_around_it(ops, dtype, M, K, J):
    """The product that adds to the residual stream prepares the RMS norm that
    follows (rmsnorm_pending), and the gate/up and the q/k/v products finish
    it: against the plain sum, the plain norm and the plain products."""
    eps = 1e-5   # J: the inner dimension of the product that adds to the stream (in pairs of 64 or not)
    h0 = rnd(M, K, seed=41) * 3
    nw = (1 + 0.2 * rnd(K, seed=42)).to(dtype)
    a, wo = rnd(M, J, dtype=dtype, seed=44), rnd(K, J, dtype=dtype, scale=0.2, seed=45)
    h64 = h0.double() + a.double() @ wo.double().T
    x64 = P.rms_norm(h64, nw.double(), eps)
    h = h0.to(DEV)
    delta = ops.linear(a.to(DEV), wo.to(DEV), may_split=True, pending=True)
    pending, left = ops.rmsnorm_pending(h, nw.to(DEV), eps, dtype, delta)
    assert isinstance(pending, ops.PendingNorm) and left is None
    torch.testing.assert_close(h.cpu().double(), h64, rtol=1e-5, atol=1e-4 if dtype == torch.float32 else 1e-2)
    torch.testing.assert_close(pending.ssq_part.sum(0)[:M].cpu().double(), h.cpu().double().pow(2).sum(-1), rtol=1e-5, atol=0)
    torch.testing.assert_close(pending.run().cpu().double(), x64, **tol(dtype, 1e-5, 2e-2))
    # gate/up with the SiLU gate
    I = 48
    g = torch.Generator().manual_seed(43)
    wg, wu = (torch.randn(I, K, generator=g) * 0.1).to(dtype), (torch.randn(I, K, generator=g) * 0.1).to(dtype)
    w = torch.stack([wg.view(-1, 8, K), wu.view(-1, 8, K)], dim=1).reshape(2 * I, K).contiguous().to(DEV)
    # What the consuming products are given: h * weight rounded to the activations' type (its agreement with
    # the plain norm was checked above), so that their own arithmetic is what the comparison below sees.
    x_in = x64 if dtype == torch.float32 else (
        pending.xs.cpu().double() / torch.sqrt(h.cpu().double().pow(2).mean(-1, keepdim=True) + eps))
    want = P.mlp(x_in, wg.double(), wu.double(), torch.eye(I, dtype=torch.float64))
    got = ops.linear_swiglu(pending, w, 8)
    torch.testing.assert_close(got.cpu().double(), want, **tol(dtype, 2e-5, 3e-2))
    # q/k/v with rotation and page write
    nh, nkv, hd, bs, n_pages, max_pos = 3, 1, 32, 8, 5, 90
    wq = (torch.randn((nh + 2 * nkv) * hd, K, generator=g) * 0.1).to(dtype)
    positions = torch.randint(0, max_pos, (M,), generator=g).to(torch.int32)
    cos_all, sin_all = P.rope_cos_sin(torch.arange(max_pos), P.rope_inv_freq(hd, 10000.0))
    table = torch.cat((cos_all[:, : hd // 2], sin_all[:, : hd // 2]), dim=-1).contiguous().to(DEV)
    slots = torch.randperm(n_pages * bs, generator=g)[:M].to(torch.int32)
    kpool = torch.zeros(n_pages, nkv, bs, hd, dtype=dtype, device=DEV)
    vpool = torch.zeros(n_pages, nkv, hd, bs, dtype=dtype, device=DEV)
    q = ops.linear_rope_kv(pending, wq.to(DEV), positions.to(DEV), table, slots.to(DEV), kpool, vpool, num_heads=nh,
                           num_kv_heads=nkv, head_dim=hd, page_size=bs)
    assert q.shape == (M, nh * hd)
    qkv = (x_in @ wq.double().T).view(M, nh + 2 * nkv, hd)
    cos, sin = P.rope_cos_sin(positions, P.rope_inv_freq(hd, 10000.0))
    rotated = P.apply_rope(qkv[:, : nh + nkv].transpose(0, 1), cos.double(), sin.double()).transpose(0, 1)
    t = tol(dtype, 2e-5, 3e-2)
    torch.testing.assert_close(q.cpu().double().view(M, nh, hd), rotated[:, :nh], **t)
    for i in range(M):
        page, off = int(slots[i]) // bs, int(slots[i]) % bs
        torch.testing.assert_close(kpool[page, :, off, :].cpu().double(), rotated[i, nh:], **t)
        torch.testing.assert_close(vpool[page, :, :, off].cpu().double(), qkv[i, nh + nkv:], **t)
    # nothing to fold the norm into: it is not handed on
    assert ops.rmsnorm_pending(h, nw.to(DEV), eps, dtype, None) == (None, None)


# ------------------------------------------------------------------------ gemm
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,N,K", [(1, 96, 64), (7, 172, 96), (33, 256, 172), (130, 1000, 200), (200, 513, 96),
                                   (64, 128, 4096), (3, 130, 33), (65, 96, 30),
                                   # few rows and an inner dimension in steps of 64: the weight-streaming kernel
                                   (1, 2048, 2048), (8, 3072, 2048), (17, 1000, 128), (64, 130, 8192), (33, 96, 64),
                                   (5, 16, 64), (48, 515, 192), (2, 128256, 64)])
def test_gemm(ops, dtype, M, N, K):
    a, w = rnd(M, K, dtype=dtype, seed=9), rnd(N, K, dtype=dtype, scale=0.05, seed=10)
    want = a.double() @ w.double().T
    bound = (a.double().abs() @ w.double().abs().T)  # size of the sum of magnitudes: the scale of rounding error
    for out_dtype in {dtype, torch.float32}:
        out = torch.empty(M, N, dtype=out_dtype, device=DEV)
        ops.gemm_nt(a.to(DEV), w.to(DEV), out)
        err = (out.cpu().double() - want).abs()
        rel = 2e-6 if dtype == torch.float32 else (1e-5 if out_dtype == torch.float32 else 1e-2)
        assert (err <= rel * bound + 1e-30).all(), f"max err {err.max()} vs bound {bound.max()}"
    acc = rnd(M, N, seed=11)
    out = acc.to(DEV)
    ops.gemm_nt(a.to(DEV), w.to(DEV), out, accumulate=True)
    err = (out.cpu().double() - (acc.double() + want)).abs()
    assert (err <= 1e-5 * (bound + acc.double().abs())).all()


def test_float_logits_of_many_rows_are_not_rounded_to_bfloat16(ops):
    """With more rows than the weight-streaming kernel takes the product goes to
    the vendor's library; asked for float results it must hand out the float
    sums, not bfloat16 values cast up (which would make near-ties of logits
    depend on the size of the batch)."""
    M, N, K = 70, 300, 256
    a, w = rnd(M, K, dtype=torch.bfloat16, seed=51), rnd(N, K, dtype=torch.bfloat16, scale=0.05, seed=52)
    want = a.double() @ w.double().T
    bound = a.double().abs() @ w.double().abs().T
    y = ops.linear(a.to(DEV), w.to(DEV), out_dtype=torch.float32)
    assert y.dtype == torch.float32
    assert ((y.cpu().double() - want).abs() <= 1e-5 * bound + 1e-30).all()


@pytest.mark.parametrize("M,N,K", [(129, 96, 64), (300, 520, 192), (257, 255, 128), (1024, 384, 320), (513, 2051, 64),
                                   (2048, 512, 1024)])
def test_bfloat16_product_of_many_rows_in_this_package(ops, M, N, K, monkeypatch):
    """The tiled kernel for prompt steps without the vendor's library (tiles of 256 tokens, loads that go
    straight to LDS into swizzled rows): all three outputs, both tile widths, against float64; rows and
    features that are no multiple of the tile, of 16 or of 4, one step of K and an odd number of them."""
    monkeypatch.setattr(ops, "LIBRARY_GEMM", False)
    a, w = rnd(M, K, dtype=torch.bfloat16, seed=71), rnd(N, K, dtype=torch.bfloat16, scale=0.05, seed=72)
    want = a.double() @ w.double().T
    bound = a.double().abs() @ w.double().abs().T
    lib = ops.core()
    try:
        for which in (1, 2, 3, 0):
            assert lib.lyp_gemm_wide(which) == 0
            for out_dtype, rel in ((torch.float32, 1e-5), (torch.bfloat16, 1e-2)):
                out = torch.full((M, N), float("nan"), dtype=out_dtype, device=DEV)
                ops.gemm_nt(a.to(DEV), w.to(DEV), out)
                err = (out.cpu().double() - want).abs()
                assert (err <= rel * bound + 1e-30).all(), (which, out_dtype, float(err.max()))
            acc = rnd(M, N, seed=73)
            out = acc.to(DEV)
            ops.gemm_nt(a.to(DEV), w.to(DEV), out, accumulate=True)
            err = (out.cpu().double() - acc.double() - want).abs()
            assert (err <= 1e-5 * bound + 2e-6 * acc.abs().double() + 1e-30).all(), (which, float(err.max()))
    finally:
        lib.lyp_gemm_wide(1)


def test_library_products_keep_one_plan_per_shape(ops):
    """The vendor's library called directly: operands that are column ranges of
    wider tensors (rows further apart than they are long), both output types,
    against the product in float64, and a plan made once per shape."""
    M, N, K = 200, 328, 136
    a_full, w_full = rnd(M, K + 24, dtype=torch.bfloat16, seed=61), rnd(N, K + 8, dtype=torch.bfloat16, scale=0.05, seed=62)
    a, w = a_full.to(DEV)[:, 8:8 + K], w_full.to(DEV)[:, :K]
    want = a.cpu().double() @ w.cpu().double().T
    bound = a.cpu().double().abs() @ w.cpu().double().abs().T
    for out_dtype, rel in ((torch.float32, 1e-5), (torch.bfloat16, 1e-2)):
        out_full = torch.zeros(M, N + 16, dtype=out_dtype, device=DEV)
        out = out_full[:, 16:]
        for _ in range(3):
            ops.library_gemm_nt(a, w, out)
        assert ((out.cpu().double() - want).abs() <= rel * bound + 1e-30).all()
        assert float(out_full[:, :16].abs().max()) == 0.0       # nothing written beside the output
    before = ops.blas().lyp_library_gemm_plans()
    ops.library_gemm_nt(a, w, torch.empty(M, N, dtype=torch.float32, device=DEV))   # other stride of the output: a new plan
    ops.library_gemm_nt(a, w, torch.empty(M, N, dtype=torch.float32, device=DEV))
    assert ops.blas().lyp_library_gemm_plans() == before + 1
    with pytest.raises(ops.KernelError, match="library gemm"):
        ops.library_gemm_nt(a.float(), w, torch.empty(M, N, dtype=torch.float32, device=DEV))


def test_library_products_chosen_by_measurement_are_checked_products(ops):
    """With tuning on (the engine's default outside the test session) a shape's first call screens
    every solution the library lists and times the fastest few; whatever wins has had its output held
    against the heuristic's first choice.  The products it leaves behind, both output types, against
    float64; and an odd number of rows that comes up after tuning is over takes the choice measured
    for its neighbour and is still the product."""
    N, K = 776, 264          # a matrix no other test multiplies: its plans are made here
    w = rnd(N, K, dtype=torch.bfloat16, scale=0.05, seed=72).to(DEV)

    def check(M, out_dtype, rel):
        a = rnd(M, K, dtype=torch.bfloat16, seed=70 + M).to(DEV)
        out = torch.empty(M, N, dtype=out_dtype, device=DEV)
        ops.library_gemm_nt(a, w, out)
        ops.library_gemm_nt(a, w, out)        # the kept plan, once more
        want = a.cpu().double() @ w.cpu().double().T
        bound = a.cpu().double().abs() @ w.cpu().double().abs().T
        assert ((out.cpu().double() - want).abs() <= rel * bound + 1e-30).all(), (M, out_dtype)
        return ops.library_gemm_solution(a, w, out)

    plans = ops.blas().lyp_library_gemm_plans()
    with ops.library_gemm_tuning(candidates=16):
        chosen = {M: check(M, torch.bfloat16, 1e-2) for M in (128, 520)}
        check(128, torch.float32, 1e-5)
    assert ops.blas().lyp_library_gemm_plans() == plans + 3 and all(c >= 0 for c in chosen.values())
    assert ops.library_gemm_rejected() >= 0
    # tuning is off again: 141 rows take what was measured at 128, 500 rows what was measured at 520
    assert check(141, torch.bfloat16, 1e-2) == chosen[128]
    assert check(500, torch.bfloat16, 1e-2) == chosen[520]


@pytest.mark.parametrize("dtype", DTYPES)
def test_tiled_product_takes_operands_that_are_column_ranges(ops, dtype, monkeypatch):
    """This package's tiled kernel with rows further apart than they are long (a column range of a
    fused output handed on as an activation), and a refusal when a row's values are not
    neighbours."""
    monkeypatch.setattr(ops, "LIBRARY_GEMM", False)
    M, N, K = 70, 96, 80
    a_full, w_full = rnd(M, K + 24, dtype=dtype, seed=71).to(DEV), rnd(N, K + 8, dtype=dtype, scale=0.1, seed=72).to(DEV)
    a, w = a_full[:, 8:8 + K], w_full[:, :K]
    out_full = torch.zeros(M, N + 16, dtype=dtype, device=DEV)
    out = out_full[:, 16:]
    ops.gemm_nt(a, w, out)
    want = a.cpu().double() @ w.cpu().double().T
    torch.testing.assert_close(out.cpu().double(), want, **tol(dtype, 2e-5, 2e-2))
    assert float(out_full[:, :16].abs().max()) == 0.0
    with pytest.raises(ops.KernelError, match="neighbours"):      # every second column: not a row of neighbours
        ops.gemm_nt(a_full[:, ::2][:, :K // 2], w_full[:, :K // 2].contiguous(), torch.empty(M, N, dtype=dtype, device=DEV))


def test_gemm_float_is_true_32_bit(ops):
    """A product whose low bits a reduced-precision matrix mode would drop."""
    K = 64
    a = torch.full((4, K), 1.0 + 2.0 ** -12)
    w = torch.full((8, K), 1.0 + 2.0 ** -11)
    out = torch.empty(4, 8, dtype=torch.float32, device=DEV)
    ops.gemm_nt(a.to(DEV), w.to(DEV), out)
    want = float(K * (1.0 + 2.0 ** -12) * (1.0 + 2.0 ** -11))
    assert abs(out.cpu()[0, 0].item() - want) < 1e-4  # a 10-bit mantissa would be off by ~0.05


# ----------------------------------------------------- rotation and page write
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,hd,bs,T", [(6, 2, 48, 8, 11), (4, 4, 16, 4, 11), (3, 1, 128, 16, 11),
                                            (8, 2, 64, 16, 75), (6, 2, 48, 8, 40)])
def test_rope_kv_write(ops, dtype, nh, nkv, hd, bs, T):
    """Few tokens take the kernel with a workgroup per token, 16 or more the one
    with 16 tokens per workgroup, which stores values of tokens in neighbouring
    slots of a page together: tokens 16..47 below are such runs (where the page
    is long enough), the others lie anywhere."""
    n_pages, max_pos = (64 + 2 * T) // bs + 2, 64
    qkv = rnd(T, (nh + 2 * nkv) * hd, dtype=dtype, seed=12)
    positions = torch.tensor(([0, 1, 2, 3, 40, 41, 42, 63, 5, 6, 7] * 7)[:T], dtype=torch.int32)
    inv_freq = P.rope_inv_freq(hd, 10000.0)
    cos_all, sin_all = P.rope_cos_sin(torch.arange(max_pos), inv_freq)
    table = torch.cat((cos_all[:, : hd // 2], sin_all[:, : hd // 2]), dim=-1).contiguous()
    slots = torch.randperm(n_pages * bs - 64, generator=torch.Generator().manual_seed(13))[:T].to(torch.int32) + 64
    if T >= 48:
        slots[16:48] = torch.arange(16, 48, dtype=torch.int32)   # two runs of 16, page by page when bs is 16
    slots[4] = -1  # "do not store"
    kpool = torch.zeros(n_pages, nkv, bs, hd, dtype=dtype, device=DEV)
    vpool = torch.zeros(n_pages, nkv, hd, bs, dtype=dtype, device=DEV)
    dev = qkv.to(DEV)
    ops.rope_kv_write(dev, positions.to(DEV), table.to(DEV), slots.to(DEV), kpool, vpool, num_heads=nh,
                      num_kv_heads=nkv, head_dim=hd, page_size=bs)
    got = dev.cpu().float().view(T, nh + 2 * nkv, hd)
    src = qkv.float().view(T, nh + 2 * nkv, hd)
    cos, sin = P.rope_cos_sin(positions, inv_freq)
    want_qk = P.apply_rope(src[:, : nh + nkv].transpose(0, 1), cos, sin).transpose(0, 1)
    t = tol(dtype, 1e-6, 1e-2)
    torch.testing.assert_close(got[:, : nh + nkv], want_qk, **t)
    torch.testing.assert_close(got[:, nh + nkv:], src[:, nh + nkv:], rtol=0, atol=0)  # values are not rotated
    torch.testing.assert_close(got[0, :nh], src[0, :nh], rtol=0, atol=0)  # position 0 is the identity
    kp, vp = kpool.cpu().float(), vpool.cpu().float()
    for i in range(T):
        if slots[i] < 0:
            continue
        page, off = int(slots[i]) // bs, int(slots[i]) % bs
        torch.testing.assert_close(kp[page, :, off, :], got[i, nh: nh + nkv], rtol=0, atol=0)
        torch.testing.assert_close(vp[page, :, :, off], got[i, nh + nkv:], rtol=0, atol=0)
    written = sum(1 for s in slots.tolist() if s >= 0)
    assert int((kp.abs().sum(-1) > 0).sum()) == written * nkv  # nothing else was touched


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,hd,rot,bs,T,has_kv", [
    (32, 8, 64, 64, 16, 8, True), (6, 2, 48, 48, 8, 1, True), (4, 4, 16, 16, 4, 19, True),
    (3, 1, 128, 32, 16, 64, True),   # only part of a head is rotated
    (5, 1, 32, 0, 16, 7, True),      # no rotation at all
    (4, 2, 64, 64, 16, 33, False),   # a layer that reads another layer's keys: query heads only
    (2, 1, 80, 40, 16, 5, True),     # a rotary size that is no multiple of 16: two kernels
])
def test_projection_with_rotation_and_page_write_in_one_kernel(ops, dtype, nh, nkv, hd, rot, bs, T, has_kv):
    """The fused q/k/v projection gives, bit for bit, what the product followed
    by the rotation and page-write kernel gives (which has its own test above)."""
    K, n_pages, max_pos = 192, 9, 300
    width = (nh + 2 * nkv) * hd if has_kv else nh * hd
    x = rnd(T, K, dtype=dtype, seed=21).to(DEV)
    w = (rnd(width, K, dtype=dtype, seed=22) * 0.3).to(DEV)
    positions = torch.randint(0, max_pos, (T,), generator=torch.Generator().manual_seed(23)).to(torch.int32).to(DEV)
    table = None
    if rot:
        cos, sin = P.rope_cos_sin(torch.arange(max_pos), P.rope_inv_freq(rot, 10000.0))
        table = torch.cat((cos[:, : rot // 2], sin[:, : rot // 2]), dim=-1).contiguous().to(DEV)
    slots = torch.randperm(n_pages * bs, generator=torch.Generator().manual_seed(24))[:T].to(torch.int32)
    slots[T // 2] = -1
    slots = slots.to(DEV)
    kw = dict(num_heads=nh, num_kv_heads=nkv, head_dim=hd, page_size=bs, has_kv=has_kv)

    def pools():
        if not has_kv:
            return None, None
        return (torch.full((n_pages, nkv, bs, hd), 7.0, dtype=dtype, device=DEV),
                torch.full((n_pages, nkv, hd, bs), 7.0, dtype=dtype, device=DEV))

    k1, v1 = pools()
    two = ops.linear(x, w, out_dtype=dtype)
    ops.rope_kv_write(two, positions, table, slots if has_kv else None, k1, v1, **kw)
    k2, v2 = pools()
    one = ops.linear_rope_kv(x, w, positions, table, slots if has_kv else None, k2, v2, **kw)
    assert torch.equal(one[:, : nh * hd], two[:, : nh * hd])
    if has_kv:
        assert torch.equal(k1, k2) and torch.equal(v1, v2)
        assert int((k2 != 7.0).any(-1).sum()) == (T - 1) * nkv  # the token without a slot stored nothing


# ------------------------------------------------------------------- attention
def paged_setup(seqs, nh, nkv, hd, bs, dtype, seed=0, n_pages=None):
    """seqs: list of (ctx_len, q_len).  Random q for the new tokens, k/v for the
    whole context, scattered over shuffled pages."""
    g = torch.Generator().manual_seed(seed)
    need = sum(-(-c // bs) for c, _ in seqs)
    n_pages = n_pages or need + 3
    perm = torch.randperm(n_pages, generator=g).tolist()
    kpool = torch.randn(n_pages, nkv, bs, hd, generator=g).to(dtype) * 3  # stale data everywhere
    vpool = torch.randn(n_pages, nkv, hd, bs, generator=g).to(dtype) * 3
    width = max(-(-c // bs) for c, _ in seqs)
    bt = torch.full((len(seqs), width), -1, dtype=torch.int32)
    qs, ks, vs, q_start = [], [], [], [0]
    for b, (ctx, ql) in enumerate(seqs):
        k = torch.randn(nkv, ctx, hd, generator=g).to(dtype)
        v = torch.randn(nkv, ctx, hd, generator=g).to(dtype)
        q = torch.randn(nh, ql, hd, generator=g).to(dtype)
        pages = [perm.pop() for _ in range(-(-ctx // bs))]
        bt[b, : len(pages)] = torch.tensor(pages, dtype=torch.int32)
        for p in range(ctx):
            kpool[pages[p // bs], :, p % bs, :] = k[:, p]
            vpool[pages[p // bs], :, :, p % bs] = v[:, p]
        qs.append(q), ks.append(k), vs.append(v)
        q_start.append(q_start[-1] + ql)
    q_flat = torch.cat([q.transpose(0, 1).reshape(q.shape[1], nh * hd) for q in qs], dim=0)
    return dict(q=q_flat, qs=qs, ks=ks, vs=vs, kpool=kpool, vpool=vpool, bt=bt,
                q_start=torch.tensor(q_start, dtype=torch.int32),
                ctx_len=torch.tensor([c for c, _ in seqs], dtype=torch.int32))


def plain_attention(s, seqs, window):
    outs = []
    for (ctx, ql), q, k, v in zip(seqs, s["qs"], s["ks"], s["vs"]):
        o = P.attention(q.double(), k.double(), v.double(), torch.arange(ctx - ql, ctx), torch.arange(ctx),
                        window=window)
        outs.append(o.transpose(0, 1).reshape(ql, -1))
    return torch.cat(outs, dim=0)


PREFILL_CASES = [
    # nh, nkv, hd, bs, window, [(ctx, q_len)]
    (4, 2, 16, 4, 0, [(5, 5), (17, 17), (33, 33)]),
    (3, 1, 32, 16, 0, [(130, 130), (9, 9), (64, 2), (70, 7)]),
    (6, 2, 48, 8, 0, [(100, 37), (65, 65), (200, 3)]),
    (8, 2, 64, 16, 0, [(300, 150), (64, 64), (129, 2)]),
    (4, 4, 128, 16, 0, [(90, 31), (17, 5)]),
    (32, 8, 64, 16, 0, [(700, 200)]),
    (5, 5, 80, 16, 0, [(40, 40)]),
    (4, 2, 32, 4, 9, [(50, 50), (33, 6), (20, 2)]),
    (2, 1, 64, 16, 40, [(200, 100), (41, 3)]),
    (16, 1, 16, 2, 0, [(23, 11)]),  # a page size that is no multiple of 4: the scalar load path
    # enough work that a workgroup takes a heavy and a light run of tokens, one after the other
    (32, 8, 64, 16, 0, [(2065, 2065)]),
    (16, 8, 32, 16, 300, [(1500, 1500), (900, 500), (65, 65), (64, 64)]),
    (8, 8, 128, 16, 0, [(2100, 2100)]),
    (2, 1, 256, 16, 0, [(100, 100), (40, 3)]),
    # larger pages: 32, 64 and 128 slots
    (8, 2, 64, 32, 0, [(700, 300), (33, 33)]),
    (4, 1, 128, 64, 0, [(500, 500), (70, 3)]),
    (8, 4, 64, 128, 200, [(900, 400)]),
    (4, 2, 32, 64, 0, [(300, 300)]),
    # three, five, six and seven query heads to a key/value head
    (24, 8, 128, 16, 0, [(300, 300), (77, 5)]),
    (5, 1, 64, 16, 0, [(200, 130)]),
    (12, 2, 64, 16, 50, [(333, 333)]),
    (7, 1, 32, 16, 0, [(150, 150)]),
]


@pytest.mark.parametrize("split,parts", [(True, 1), (False, 1), (True, 3), (False, 4)],
                         ids=["split", "whole", "split-3-parts", "4-parts"])
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("case", PREFILL_CASES, ids=[str(c[:5]) for c in PREFILL_CASES])
def test_attention_prefill(ops, dtype, case, split, parts):
    """``split``: a small launch may give a tile's keys to two sets of waves in turn.  ``parts``: every
    tile's keys in that many runs, for workgroups of their own, put together by a second kernel."""
    nh, nkv, hd, bs, window, seqs = case
    s = paged_setup(seqs, nh, nkv, hd, bs, dtype, seed=hd + bs)
    tile_seq, tile_q0 = [], []
    for b, (_, ql) in enumerate(seqs):
        for q0 in range(0, ql, 64):
            tile_seq.append(b), tile_q0.append(q0)
    out = torch.full((s["q"].shape[0], nh * hd), float("nan"), dtype=dtype, device=DEV)
    work = {}
    if parts > 1:
        n = len(tile_seq) * 64 * nh * parts
        work = dict(parts=parts, part_o=torch.full((n * hd,), float("nan"), device=DEV),
                    part_ml=torch.full((n * 2,), float("nan"), device=DEV))
    ops.attn_prefill(s["q"].to(DEV), out, s["kpool"].to(DEV), s["vpool"].to(DEV), s["bt"].to(DEV),
                     s["q_start"].to(DEV), s["ctx_len"].to(DEV), torch.tensor(tile_seq, dtype=torch.int32, device=DEV),
                     torch.tensor(tile_q0, dtype=torch.int32, device=DEV), len(tile_seq), num_heads=nh,
                     num_kv_heads=nkv, head_dim=hd, window=window, split=split, **work)
    want = plain_attention(s, seqs, window)
    torch.testing.assert_close(out.cpu().double(), want, **tol(dtype, 2e-5, 2e-2))


@pytest.mark.parametrize("variant", ["two sets of waves", "keys in 4 runs", "paired tiles"])
def test_bfloat16_prefill_kernel_rounds_like_one_rounding(ops, variant):
    """The kernel that exists in bfloat16 only (16x16x32 products, probabilities rounded to
    bfloat16 before they meet the values) in each of its forms, on inputs that are bfloat16
    values already, against the formula in float64: what is measured is the kernel's own rounding,
    and it stays inside 1e-2 (the probabilities' 8 bits, averaged over the keys)."""
    nh, nkv, hd, bs = 32, 8, 64, 16
    seqs = [(2065, 2065)] if variant == "paired tiles" else [(700, 200), (300, 64)]
    s = paged_setup(seqs, nh, nkv, hd, bs, torch.bfloat16, seed=17)
    tile_seq, tile_q0 = [], []
    for b, (_, ql) in enumerate(seqs):
        for q0 in range(0, ql, 64):
            tile_seq.append(b), tile_q0.append(q0)
    out = torch.full((s["q"].shape[0], nh * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
    work = dict(split=variant == "two sets of waves")
    if variant == "keys in 4 runs":
        n = len(tile_seq) * 64 * nh * 4
        work.update(parts=4, part_o=torch.full((n * hd,), float("nan"), device=DEV),
                    part_ml=torch.full((n * 2,), float("nan"), device=DEV))
    ops.attn_prefill(s["q"].to(DEV), out, s["kpool"].to(DEV), s["vpool"].to(DEV), s["bt"].to(DEV),
                     s["q_start"].to(DEV), s["ctx_len"].to(DEV), torch.tensor(tile_seq, dtype=torch.int32, device=DEV),
                     torch.tensor(tile_q0, dtype=torch.int32, device=DEV), len(tile_seq), num_heads=nh,
                     num_kv_heads=nkv, head_dim=hd, pair=variant == "paired tiles", **work)
    torch.testing.assert_close(out.cpu().double(), plain_attention(s, seqs, 0), rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("M,N,K", [(8, 3072, 2048), (33, 2048, 2048), (64, 2048, 8192), (48, 3072, 2048), (40, 2048, 1024)])
def test_bfloat16_few_rows_product_rounds_once(ops, M, N, K):
    """The weight-streaming product's 16x16x32 path (one and two row tiles per workgroup, partial
    sums over slices of K) on bfloat16 inputs against float64: float sums, one rounding at the end."""
    a, w = rnd(M, K, dtype=torch.bfloat16, seed=31), rnd(N, K, dtype=torch.bfloat16, scale=0.05, seed=32)
    want = a.double() @ w.double().T
    scale = float(want.abs().max())
    y = ops.linear(a.to(DEV), w.to(DEV))
    assert float((y.cpu().double() - want).abs().max()) <= 2.0 ** -8 * scale        # the one rounding to bfloat16
    parts = ops.linear(a.to(DEV), w.to(DEV), may_split=True)
    total = ops.sum_parts(parts, torch.float32)
    # float partial sums where this package's kernel took the product in slices; one rounding to
    # bfloat16 where the launch would have needed several rounds of workgroups and the library took it
    limit = 1e-5 if parts.dim() == 3 else 2.0 ** -8
    assert float((total.cpu().double() - want).abs().max()) <= limit * scale
    assert parts.dim() == 3 or M > 40      # (the larger ones are more than one small round of workgroups)


def test_attention_prefill_plan(ops):
    plan = lambda tiles, keys, dt=torch.bfloat16, bs=16: ops.attn_prefill_plan(tiles, keys, 32, 8, 64, dt, bs)
    assert plan(32, 2048) == 1                 # a whole prompt: enough workgroups as it is
    assert plan(8, 8192) == 2                  # 512 new tokens at the end of 8192
    assert plan(1, 8192) > plan(8, 8192)       # fewer tokens, more runs
    assert plan(8, 512) == 1                   # few keys: nothing to cut
    assert plan(8, 8192, torch.float32) == 1 and plan(8, 8192, bs=4) == 1   # the other kernel has no parts


DECODE_CASES = [
    (4, 2, 16, 4, 0, [1, 15, 64, 65]),
    (3, 1, 32, 16, 0, [300, 1, 129]),
    (32, 8, 64, 16, 0, [1000, 17]),
    (6, 2, 48, 8, 0, [48, 200]),
    (4, 1, 128, 16, 0, [513]),
    (40, 2, 32, 16, 0, [77]),        # more than 16 query heads per key/value head
    (4, 2, 32, 4, 9, [50, 5, 9, 10]),
    (2, 1, 64, 16, 100, [700, 64]),
    (16, 1, 16, 2, 0, [23]),
    (8, 2, 64, 32, 0, [700, 33]),     # larger pages
    (4, 1, 128, 64, 0, [500, 1]),
    (8, 4, 64, 128, 200, [900, 129]),
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("case", DECODE_CASES, ids=[str(c[:5]) for c in DECODE_CASES])
def test_attention_decode(ops, dtype, case):
    nh, nkv, hd, bs, window, ctxs = case
    seqs = [(c, 1) for c in ctxs]
    s = paged_setup(seqs, nh, nkv, hd, bs, dtype, seed=hd + bs + 1)
    n = len(seqs)
    part = ops.attn_decode_plan(n, max(ctxs), nh, nkv, hd)
    max_parts = -(-max(ctxs) // part)
    part_o = torch.full((n * nh * max_parts * hd,), float("nan"), device=DEV)
    part_ml = torch.full((n * nh * max_parts * 2,), float("nan"), device=DEV)
    out = torch.full((n, nh * hd), float("nan"), dtype=dtype, device=DEV)
    # the requests in shuffled order through dec_seqs
    order = list(reversed(range(n)))
    ops.attn_decode(s["q"].to(DEV), out, s["kpool"].to(DEV), s["vpool"].to(DEV), s["bt"].to(DEV),
                    s["q_start"].to(DEV), s["ctx_len"].to(DEV), torch.tensor(order, dtype=torch.int32, device=DEV), n,
                    part_o, part_ml, max_parts, part, num_heads=nh, num_kv_heads=nkv, head_dim=hd, window=window)
    want = plain_attention(s, seqs, window)
    torch.testing.assert_close(out.cpu().double(), want, **tol(dtype, 2e-5, 2e-2))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", ["prefill", "decode"])
def test_attention_finds_one_far_key(ops, dtype, kind):
    """Among 900 keys one, far back, matches the query strongly: the output is
    that key's value.  Random data would hide a kernel that drops distant keys
    or a page."""
    nh, nkv, hd, bs, ctx, far = 4, 2, 64, 16, 900, 37
    ql = 1 if kind == "decode" else 5
    seqs = [(ctx, ql)]
    s = paged_setup(seqs, nh, nkv, hd, bs, dtype, seed=5)
    k = s["ks"][0]
    k[:, far] = 4.0
    s["qs"][0][:] = 4.0   # score with the far key: 16 * 64 / 8 = 128; with the others ~ N(0, 32)
    pages = s["bt"][0].tolist()
    s["kpool"][pages[far // bs], :, far % bs, :] = k[:, far]
    s["q"] = torch.cat([q.transpose(0, 1).reshape(q.shape[1], nh * hd) for q in s["qs"]], dim=0)
    out = torch.empty((ql, nh * hd), dtype=dtype, device=DEV)
    args = (s["q"].to(DEV), out, s["kpool"].to(DEV), s["vpool"].to(DEV), s["bt"].to(DEV), s["q_start"].to(DEV),
            s["ctx_len"].to(DEV))
    kw = dict(num_heads=nh, num_kv_heads=nkv, head_dim=hd)
    if kind == "decode":
        part = ops.attn_decode_plan(1, ctx, nh, nkv, hd)
        mp = -(-ctx // part)
        ops.attn_decode(*args, None, 1, torch.empty(nh * mp * hd, device=DEV), torch.empty(nh * mp * 2, device=DEV),
                        mp, part, **kw)
    else:
        ops.attn_prefill(*args, torch.zeros(1, dtype=torch.int32, device=DEV),
                         torch.zeros(1, dtype=torch.int32, device=DEV), 1, **kw)
    v_far = s["vs"][0][:, far].float()  # [nkv, hd]
    want = v_far.repeat_interleave(nh // nkv, dim=0).reshape(1, nh * hd).expand(ql, -1)
    torch.testing.assert_close(out.cpu().float(), want, rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", ["prefill", "decode"])
@pytest.mark.parametrize("window", [48, 50, 64, 129])   # the edge at a page's first slot, inside a page, a tile wide
def test_attention_at_the_edge_of_the_window(ops, dtype, kind, window):
    """The last key inside the window and the first one outside both match the
    query strongly, the outer one more so: the output must be the inner key's
    value.  A mask that is off by one at the edge gives the other value; random
    data would change the output by a few hundredths only."""
    nh, nkv, hd, bs, ctx = 4, 2, 64, 16, 400
    ql = 1 if kind == "decode" else 3
    seqs = [(ctx, ql)]
    s = paged_setup(seqs, nh, nkv, hd, bs, dtype, seed=6)
    k, pages = s["ks"][0], s["bt"][0].tolist()
    s["qs"][0][:] = 0.0
    out_key = {}
    for i in range(ql):                      # every new token has an edge of its own
        pos = ctx - ql + i
        inner, outer = pos - window + 1, pos - window
        out_key[i] = inner
        s["qs"][0][:, i, i] = 8.0            # token i looks at dimension i alone
        k[:, :, i] = 0.0
        k[:, inner, i] = 6.0                 # score 8 * 6 / 8 = 6 over zeros elsewhere ... times log-odds of 400 keys
        k[:, outer, i] = 12.0                # the outer one would win if it were visible
    for p in range(ctx):
        s["kpool"][pages[p // bs], :, p % bs, :] = k[:, p]
    # pages that the window has passed for every new token are gone from the table, as the cache
    # manager leaves it (-1), and hold something else by now
    gone = (ctx - ql - window + 1) // bs
    for page in pages[:gone]:
        s["kpool"][page] = 50.0
        s["vpool"][page] = 50.0
    s["bt"][0, :gone] = -1
    s["q"] = torch.cat([q.transpose(0, 1).reshape(q.shape[1], nh * hd) for q in s["qs"]], dim=0)
    out = torch.empty((ql, nh * hd), dtype=dtype, device=DEV)
    args = (s["q"].to(DEV), out, s["kpool"].to(DEV), s["vpool"].to(DEV), s["bt"].to(DEV), s["q_start"].to(DEV),
            s["ctx_len"].to(DEV))
    kw = dict(num_heads=nh, num_kv_heads=nkv, head_dim=hd, window=window)
    if kind == "decode":
        part = ops.attn_decode_plan(1, ctx, nh, nkv, hd)
        mp = -(-ctx // part)
        ops.attn_decode(*args, None, 1, torch.empty(nh * mp * hd, device=DEV), torch.empty(nh * mp * 2, device=DEV),
                        mp, part, **kw)
    else:
        ops.attn_prefill(*args, torch.zeros(1, dtype=torch.int32, device=DEV),
                         torch.zeros(1, dtype=torch.int32, device=DEV), 1, **kw)
    want = plain_attention(s, seqs, window)
    torch.testing.assert_close(out.cpu().double(), want, **tol(dtype, 2e-5, 2e-2))
    # and the plain reference itself is dominated by the inner key, not the outer one
    for i in range(ql):
        v_in = s["vs"][0][:, out_key[i]].double().repeat_interleave(nh // nkv, dim=0).reshape(-1)
        v_out = s["vs"][0][:, out_key[i] - 1].double().repeat_interleave(nh // nkv, dim=0).reshape(-1)
        assert (want[i] - v_in).abs().max() < 0.5 * (want[i] - v_out).abs().max()


# ------------------------------------------------ attention at long contexts
def paged_setup_long(seqs, nh, nkv, hd, bs, dtype, seed=0, q_scale=4.0):
    """``paged_setup`` for contexts of thousands of tokens: built on the device, whole pages at a
    time.  Queries are scaled so that the softmax is peaked (a handful of keys among thousands carry
    a row's weight): a run or a partition of keys that is dropped, read twice or merged wrongly
    then moves the result far beyond the tolerance, which a flat softmax would not."""
    g = torch.Generator(device=DEV).manual_seed(seed)
    cpu_g = torch.Generator().manual_seed(seed)
    need = sum(-(-c // bs) for c, _ in seqs)
    n_pages = need + 5
    perm = torch.randperm(n_pages, generator=cpu_g)
    rand = lambda *shape: torch.randn(*shape, generator=g, device=DEV)
    kpool = (rand(n_pages, nkv, bs, hd) * 3).to(dtype)     # stale data everywhere
    vpool = (rand(n_pages, nkv, hd, bs) * 3).to(dtype)
    width = max(-(-c // bs) for c, _ in seqs)
    bt = torch.full((len(seqs), width), -1, dtype=torch.int32)
    qs, ks, vs, q_start, at = [], [], [], [0], 0
    for b, (ctx, ql) in enumerate(seqs):
        npg = -(-ctx // bs)
        pages = perm[at:at + npg]
        at += npg
        bt[b, :npg] = pages.to(torch.int32)
        k = (rand(nkv, npg * bs, hd)).to(dtype)            # the tail past ctx is stale data too
        v = (rand(nkv, npg * bs, hd)).to(dtype)
        q = (rand(nh, ql, hd) * q_scale).to(dtype)
        kpool[pages.to(DEV)] = k.view(nkv, npg, bs, hd).permute(1, 0, 2, 3)
        vpool[pages.to(DEV)] = v.view(nkv, npg, bs, hd).permute(1, 0, 3, 2)
        qs.append(q.cpu()), ks.append(k[:, :ctx].cpu()), vs.append(v[:, :ctx].cpu())
        q_start.append(q_start[-1] + ql)
    q_flat = torch.cat([q.transpose(0, 1).reshape(q.shape[1], nh * hd) for q in qs], dim=0)
    return dict(q=q_flat, qs=qs, ks=ks, vs=vs, kpool=kpool, vpool=vpool, bt=bt,
                q_start=torch.tensor(q_start, dtype=torch.int32),
                ctx_len=torch.tensor([c for c, _ in seqs], dtype=torch.int32))


def plain_attention_by_group(s, seqs):
    """The plain attention, one key/value head at a time (a whole request's scores would not fit)."""
    outs = []
    for (ctx, ql), q, k, v in zip(seqs, s["qs"], s["ks"], s["vs"]):
        nh, nkv = q.shape[0], k.shape[0]
        grp = nh // nkv
        heads = [P.attention(q[j * grp:(j + 1) * grp].double(), k[j:j + 1].double(), v[j:j + 1].double(),
                             torch.arange(ctx - ql, ctx), torch.arange(ctx)) for j in range(nkv)]
        outs.append(torch.cat(heads, dim=0).transpose(0, 1).reshape(ql, -1))
    return torch.cat(outs, dim=0)


def run_decode(ops, s, n, nh, nkv, hd, max_ctx, dtype):
    """The split kernel as the attention part launches it: partition size from the plan for this
    many requests and this bound on the context."""
    part = ops.attn_decode_plan(n, max_ctx, nh, nkv, hd)
    max_parts = -(-max_ctx // part)
    part_o = torch.full((n * nh * max_parts * hd,), float("nan"), device=DEV)
    part_ml = torch.full((n * nh * max_parts * 2,), float("nan"), device=DEV)
    out = torch.full((n, nh * hd), float("nan"), dtype=dtype, device=DEV)
    ops.attn_decode(s["q"].to(DEV), out, s["kpool"], s["vpool"], s["bt"].to(DEV), s["q_start"].to(DEV),
                    s["ctx_len"].to(DEV), None, n, part_o, part_ml, max_parts, part, num_heads=nh, num_kv_heads=nkv,
                    head_dim=hd)
    return out, part, max_parts


def run_prefill(ops, s, seqs, nh, nkv, hd, bs, dtype):
    """The prefill kernel as the attention part launches it: tiles sorted by the keys they see, the
    keys of few new tokens cut into the runs the plan says."""
    tiles = sorted((ctx - ql + min(ql, q0 + 64), b, q0) for b, (ctx, ql) in enumerate(seqs) for q0 in range(0, ql, 64))
    tile_seq = torch.tensor([t[1] for t in tiles], dtype=torch.int32, device=DEV)
    tile_q0 = torch.tensor([t[2] for t in tiles], dtype=torch.int32, device=DEV)
    few, many = tiles[0][0], tiles[-1][0]
    parts = ops.attn_prefill_plan(len(tiles), many, nh, nkv, hd, dtype, bs)
    work = {}
    if parts > 1:
        n = len(tiles) * 64 * nh * parts
        work = dict(parts=parts, part_o=torch.full((n * hd,), float("nan"), device=DEV),
                    part_ml=torch.full((n * 2,), float("nan"), device=DEV))
    out = torch.full((s["q"].shape[0], nh * hd), float("nan"), dtype=dtype, device=DEV)
    ops.attn_prefill(s["q"].to(DEV), out, s["kpool"], s["vpool"], s["bt"].to(DEV), s["q_start"].to(DEV),
                     s["ctx_len"].to(DEV), tile_seq, tile_q0, len(tiles), num_heads=nh, num_kv_heads=nkv, head_dim=hd,
                     pair=2 * few <= many, **work)
    return out, parts


LONG_DECODE_CASES = [
    # heads, key/value heads, head size, page size, bound on the context, contexts
    (32, 8, 64, 16, 8192, [8192]),                                             # the benchmark's shape, batch 1
    (32, 8, 64, 16, 8192, [8192, 8191, 8177, 8166, 8130, 8100, 8065, 8129]),   # and batch 8, contexts as they grow
    (24, 8, 128, 16, 8192, [8192]),
    (24, 8, 128, 16, 8192, [8192, 8000, 8111, 7777, 8190, 8050, 8001, 8160]),
    (32, 8, 64, 16, 32768, [32768]),
    (32, 8, 64, 16, 32768, [32768, 32700, 30000, 32767, 31000, 32000, 29000, 32100]),
    (24, 8, 128, 16, 32768, [32768]),
    (32, 8, 64, 16, 16384, [8193, 9000]),                                      # a recorded step's bound above every context
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("case", LONG_DECODE_CASES, ids=[f"{c[0]}/{c[1]}x{c[2]}-{c[4]}-b{len(c[5])}" for c in LONG_DECODE_CASES])
def test_attention_decode_at_the_benchmarks_contexts(ops, dtype, case):
    """Contexts of 8,192 and 32,768 keys, batch 1 and 8, the 1B shape's heads (32 over 8, 64 wide)
    and the 3B shape's (24 over 8, 128 wide), with the partition size that the plan gives for exactly
    these launches: many partitions per request, block tables 512 to 2,048 entries wide."""
    nh, nkv, hd, bs, bound, ctxs = case
    seqs = [(c, 1) for c in ctxs]
    s = paged_setup_long(seqs, nh, nkv, hd, bs, dtype, seed=hd + len(ctxs))
    out, part, max_parts = run_decode(ops, s, len(seqs), nh, nkv, hd, bound, dtype)
    assert max_parts >= 4, "the case is meant to be cut into several partitions"
    want = plain_attention_by_group(s, seqs)
    assert float(want.abs().max()) > 0.5          # peaked: single keys show in the result
    torch.testing.assert_close(out.cpu().double(), want, **tol(dtype, 3e-5, 2e-2))


LONG_PREFILL_CASES = [
    (32, 8, 64, 16, [(8192, 512)]),
    (32, 8, 64, 16, [(8192, 64)]),
    (24, 8, 128, 16, [(8192, 512)]),
    (24, 8, 128, 16, [(8192, 64)]),
    (32, 8, 64, 16, [(8192, 300), (4100, 100), (9000, 2)]),
    (32, 8, 64, 16, [(8300, 40)]),
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("case", LONG_PREFILL_CASES, ids=[f"{c[0]}/{c[1]}x{c[2]}-{c[4]}" for c in LONG_PREFILL_CASES])
def test_attention_prefill_of_a_portion_over_8192_keys(ops, dtype, case):
    """512 and 64 new tokens at the end of 8,192 keys, with the runs of keys the plan gives."""
    nh, nkv, hd, bs, seqs = case
    s = paged_setup_long(seqs, nh, nkv, hd, bs, dtype, seed=hd + seqs[0][1])
    out, parts = run_prefill(ops, s, seqs, nh, nkv, hd, bs, dtype)
    if dtype == torch.bfloat16 and len(seqs) == 1:
        assert parts > 1, "few tokens over many keys were meant to be cut into runs"
    want = plain_attention_by_group(s, seqs)
    assert float(want.abs().max()) > 0.5
    torch.testing.assert_close(out.cpu().double(), want, **tol(dtype, 3e-5, 2e-2))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", ["prefill", "decode"])
@pytest.mark.parametrize("nh,nkv,hd", [(32, 8, 64), (24, 8, 128)])
def test_attention_finds_a_key_anywhere_in_8192(ops, dtype, kind, nh, nkv, hd):
    """Eight requests of about 8,192 keys; in each, one key matches the queries strongly, and each
    has it elsewhere: the first key, the last, both sides of a partition's edge and of a page's, the
    middle.  Every output must be that key's value, which a partition, a run or a table entry that
    is skipped or read for the wrong request cannot give."""
    bs = 16
    ql = 1 if kind == "decode" else 3
    ctxs = [8192, 8191, 8177, 8166, 8130, 8100, 8065, 8129]
    seqs = [(c, ql) for c in ctxs]
    s = paged_setup_long(seqs, nh, nkv, hd, bs, dtype, seed=9, q_scale=1.0)
    part = ops.attn_decode_plan(len(seqs), 8192, nh, nkv, hd)
    far = [0, ctxs[1] - ql, part - 1, part, 4095, 4096, 3 * part + 17, ctxs[7] // 2]
    for b, f in enumerate(far):
        s["qs"][b][:] = 4.0          # score with the planted key: 16 hd / sqrt(hd); with the others ~ N(0, 16)
        page = int(s["bt"][b, f // bs])
        s["kpool"][page, :, f % bs, :] = 4.0
    s["q"] = torch.cat([q.transpose(0, 1).reshape(q.shape[1], nh * hd) for q in s["qs"]], dim=0)
    if kind == "decode":
        out, _, _ = run_decode(ops, s, len(seqs), nh, nkv, hd, 8192, dtype)
    else:
        out, _ = run_prefill(ops, s, seqs, nh, nkv, hd, bs, dtype)
    for b, f in enumerate(far):
        v_far = s["vs"][b][:, f].float()                                   # [nkv, hd]
        want = v_far.repeat_interleave(nh // nkv, dim=0).reshape(1, nh * hd).expand(ql, -1)
        got = out[b * ql:(b + 1) * ql].cpu().float()
        torch.testing.assert_close(got, want, rtol=1e-2, atol=1e-2, msg=lambda m: f"request {b}, key {f}: {m}")


# ----------------------------------------------------------------- output head
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,V,K", [(1, 1003, 128), (8, 32000, 192), (16, 515, 64), (11, 2051, 256), (3, 128256, 64),
                                   (5, 5003, 576), (2, 1003, 1344), (7, 2051, 1024), (4, 50, 512), (3, 1003, 4672),
                                   (17, 1003, 128), (24, 515, 1344), (32, 2051, 2048), (29, 5003, 64), (20, 300, 2304)])
def test_output_head_logits_and_row_maxima(ops, dtype, M, V, K, monkeypatch):
    """The head's own kernels (few long-lived waves walking the matrix): float logits against the
    product in float64, and per row the pieces' maxima: the largest of them is the row's largest
    logit at the first place it stands.  Vocabularies that are no multiple of 16 or of 4; 1 to 16
    rows; few workgroups (every wave walks many row blocks) and many, also more waves than blocks
    of rows; widths of fewer chunks of 64 than a wave of the bfloat16 kernel asks for ahead, of
    exactly as many, of twice as many, and of a number that is no multiple of it; a width whose
    activations do not fit LDS (bfloat16 then takes the kernel that reads them from the cache).
    17 to 32 rows: bfloat16 takes the same kernel with two blocks of 16 tokens while their activations
    fit LDS; 32-bit, and a width beyond that, go to the general products and bring no row maxima."""
    x = rnd(M, K, dtype=dtype, seed=81)
    w = rnd(V, K, dtype=dtype, scale=0.2, seed=82)
    w[V // 3] = w[7]                                   # two equal logits in every row: the first one is to win
    want = x.double() @ w.double().T
    for blocks in (8, 512):
        monkeypatch.setattr(ops, "LM_HEAD_BLOCKS", blocks)
        out, maxima = ops.lm_head(x.to(DEV), w.to(DEV))
        if M > 16:
            assert (maxima is not None) == (dtype == torch.bfloat16 and K <= 2296), (M, K, dtype)
        if K <= 2048:
            torch.testing.assert_close(out.cpu().double(), want, **tol(dtype, 2e-5, 1e-2))
        else:   # a long sum: held to the size of what is added up, as the products' own test does
            bound = x.double().abs() @ w.double().abs().T
            assert ((out.cpu().double() - want).abs() <= (2e-6 if dtype == torch.float32 else 1e-5) * bound).all()
        if maxima is None:
            continue
        cand = maxima.cpu()
        assert cand.shape[0] == M and cand.shape[2] == 2 and cand.shape[1] <= blocks
        values, places = cand[..., 0].contiguous().view(torch.float32), cand[..., 1]
        got = out.cpu()
        for m in range(M):
            best = int(values[m].argmax())
            top = float(got[m].max())
            assert float(values[m, best]) == top
            first = int((got[m] == top).nonzero()[0])
            assert int(places[m][values[m] == top].min()) == first
        # the sampler takes them: greedy and drawn tokens equal those found with a pass over the row
        R = M
        temperature = torch.tensor(([0.0, 0.9, 1.2] * R)[:R]).to(DEV)
        top_k = torch.tensor(([-1, 40, -1] * R)[:R], dtype=torch.int32).to(DEV)
        top_p = torch.tensor(([1.0, 1.0, 0.8] * R)[:R]).to(DEV)
        u = torch.rand(R, generator=torch.Generator().manual_seed(3)).to(DEV)
        a, b = torch.empty(R, dtype=torch.int32, device=DEV), torch.empty(R, dtype=torch.int32, device=DEV)
        ops.sample(out, temperature, top_k, top_p, u, a, row_maxima=maxima)
        ops.sample(out, temperature, top_k, top_p, u, b, ops.sample_workspace(R, DEV))   # with a pass over the row
        assert a.tolist() == b.tolist()
        assert a[0] == int(got[0].argmax())


# --------------------------------------------------------------------- sampler
def test_sampler_greedy_and_draws(ops):
    V = 1003
    g = torch.Generator().manual_seed(3)
    logits = torch.randn(6, V, generator=g) * 3
    logits[1, 500] = logits[1, 7] = logits[1].max() + 1  # a tie: the first index wins
    temperature = torch.tensor([0.0, 0.0, 0.8, 1.3, 0.7, 1.0])
    top_k = torch.tensor([-1, -1, -1, 40, -1, 5], dtype=torch.int32)
    top_p = torch.tensor([1.0, 1.0, 1.0, 1.0, 0.6, 0.9])
    for u_val in (0.0, 0.137, 0.5, 0.77, 0.999):
        u = torch.full((6,), u_val)
        out = torch.empty(6, dtype=torch.int32, device=DEV)
        work = ops.sample_workspace(6, DEV) if u_val > 0.4 else None   # both ways of finding the maximum
        mirror = torch.full((6,), -5, dtype=torch.int32).pin_memory() if u_val > 0.1 else None
        ops.sample(logits.to(DEV), temperature.to(DEV), top_k.to(DEV), top_p.to(DEV), u.to(DEV), out, work, mirror=mirror)
        got = out.cpu().tolist()     # waits for the kernel: the pinned mirror then holds the same tokens
        assert mirror is None or mirror.tolist() == got
        assert got[0] == P.greedy(logits[0])
        assert got[1] == 7
        for r in range(2, 6):
            probs = P.sample_filter(logits[r], float(temperature[r]), int(top_k[r]), float(top_p[r]))
            assert probs[got[r]] > 0, f"row {r}: token {got[r]} was filtered out"
            cdf = torch.cumsum(probs, 0)
            lo = float(cdf[got[r]] - probs[got[r]])
            assert lo - 1e-5 <= u_val <= float(cdf[got[r]]) + 1e-5, f"row {r}: u={u_val} not in [{lo}, {float(cdf[got[r]])}]"


def test_sampler_writes_a_token_for_rows_without_a_largest_logit(ops):
    """Rows of NaN or of -inf only (broken weights, an overflow) have no largest logit; what the
    sampler writes is still a token of the vocabulary, which the next step can look up, and rows
    beside them are not disturbed.  With and without the pass that finds the maxima first, and with
    the output head's candidates."""
    V, K = 2051, 64
    g = torch.Generator().manual_seed(5)
    logits = torch.randn(6, V, generator=g)
    logits[1] = float("nan")
    logits[2] = float("-inf")
    logits[4] = float("nan")
    logits[4, 77] = 1.5                                  # one logit that compares: it is the row's choice
    temperature = torch.tensor([0.0, 0.0, 0.9, 0.8, 0.0, 1.1])
    top_k = torch.tensor([-1, -1, 10, -1, -1, 20], dtype=torch.int32)
    top_p = torch.tensor([1.0, 1.0, 0.9, 1.0, 1.0, 0.7])
    u = torch.full((6,), 0.42)
    for work in (None, ops.sample_workspace(6, DEV)):
        out = torch.full((6,), -1, dtype=torch.int32, device=DEV)
        ops.sample(logits.to(DEV), temperature.to(DEV), top_k.to(DEV), top_p.to(DEV), u.to(DEV), out, work)
        got = out.cpu().tolist()
        assert all(0 <= t < V for t in got), got
        assert got[0] == P.greedy(logits[0]) and got[1] == 0 and got[2] == 0 and got[4] == 77
        # the same rows drawn from, with and without cut-offs: still a token, and the one logit that compares
        for tk, tp in ((-1, 1.0), (5, 1.0), (-1, 0.5), (7, 0.3)):
            hot = torch.full((6,), 0.8)
            ops.sample(logits.to(DEV), hot.to(DEV), torch.full((6,), tk, dtype=torch.int32, device=DEV),
                       torch.full((6,), tp, device=DEV), u.to(DEV), out, work)
            got = out.cpu().tolist()
            assert all(0 <= t < V for t in got), (tk, tp, got)
            assert got[4] == 77, (tk, tp, got)
    # through the head's kernel: activations of NaN give rows of NaN logits and candidates without a place
    x = rnd(3, K, dtype=torch.bfloat16, seed=7)
    x[1] = float("nan")
    w = rnd(V, K, dtype=torch.bfloat16, scale=0.2, seed=8)
    head, maxima = ops.lm_head(x.to(DEV), w.to(DEV))
    assert maxima is not None
    out = torch.full((3,), -1, dtype=torch.int32, device=DEV)
    z = torch.zeros(3, device=DEV)
    ops.sample(head, z, torch.full((3,), -1, dtype=torch.int32, device=DEV), torch.ones(3, device=DEV), z, out,
               row_maxima=maxima)
    got = out.cpu().tolist()
    assert got[1] == 0 and got[0] == int(head[0].argmax()) and got[2] == int(head[2].argmax())


def _row(kind, V, g):
    if kind == "peaked":       # as a trained model's: a few tokens stand out
        x = torch.randn(V, generator=g) * 2.5
        x[torch.randperm(V, generator=g)[:20]] += 9.0
        return x
    if kind == "flat":         # as random weights give: everything within a few units
        return torch.randn(V, generator=g) * 0.3
    if kind == "ties":         # many equal values, also at the cut-offs
        return torch.randint(0, 6, (V,), generator=g).float() * 0.5
    if kind == "masked":       # most tokens ruled out beforehand
        x = torch.randn(V, generator=g)
        x[torch.rand(V, generator=g) < 0.9] = float("-inf")
        return x
    if kind == "far":          # most tokens more than 32 from the largest: the last bucket
        x = torch.randn(V, generator=g) - 60.0
        x[torch.randperm(V, generator=g)[:30]] += 60.0
        return x
    raise ValueError(kind)


@pytest.mark.parametrize("kind", ["peaked", "flat", "ties", "masked", "far"])
@pytest.mark.parametrize("V", [1003, 32000, 128256])
def test_sampler_cut_offs_against_the_sorted_reference(ops, V, kind):
    """64 draws at evenly spread uniforms for several (temperature, top-k, top-p): every token must
    be one that the plain (sorting) filter keeps, and sit where the uniform falls in the plain
    cumulative distribution.  A kept set that is off by one token shifts that distribution."""
    g = torch.Generator().manual_seed(V % 1000 + len(kind))
    x = _row(kind, V, g)
    n = 64
    rows = x.expand(n, V).contiguous().to(DEV)
    u = ((torch.arange(n) + 0.37) / n).float()
    work = ops.sample_workspace(n, DEV)
    for temp, tk, tp in [(0.8, -1, 1.0), (1.0, 40, 1.0), (0.7, -1, 0.9), (1.3, 200, 0.6), (1.0, V - 3, 0.999),
                         (0.9, 1, 0.5), (1.0, 3000, 1.0)]:
        tk = min(tk, V)
        if kind == "ties" and tp < 1.0:
            continue   # which of the equal tokens at the cut-off stay is the sort's whim there; here all of them do
        out = torch.empty(n, dtype=torch.int32, device=DEV)
        ops.sample(rows, torch.full((n,), temp).to(DEV), torch.full((n,), tk, dtype=torch.int32).to(DEV),
                   torch.full((n,), tp).to(DEV), u.to(DEV), out, work)
        got = out.cpu().tolist()
        probs = P.sample_filter(x, temp, tk, tp)
        cdf = torch.cumsum(probs, 0)
        for r in range(n):
            t = got[r]
            assert probs[t] > 0, f"{kind} V={V} T={temp} k={tk} p={tp}: token {t} is not in the kept set"
            lo, hi = float(cdf[t] - probs[t]), float(cdf[t])
            assert lo - 2e-5 <= float(u[r]) <= hi + 2e-5, \
                f"{kind} V={V} T={temp} k={tk} p={tp}: u={float(u[r])} outside [{lo}, {hi}] of token {t}"


def test_table_from_pinned_memory(ops):
    """A table of integers read from pinned host memory by the kernel itself, a
    few words of it replaced by values that only the device holds."""
    g = torch.Generator().manual_seed(8)
    src = torch.randint(-5, 10 ** 6, (1000,), generator=g, dtype=torch.int32).pin_memory()
    dst = torch.full((1000,), -9, dtype=torch.int32, device=DEV)
    ops.table_load(src, dst)
    assert torch.equal(dst.cpu(), src)
    patch = torch.arange(100, 107, dtype=torch.int32, device=DEV)
    src[:] = src + 1                       # a later step's table in the same buffer
    ops.table_load(src, dst, patch, 13)
    want = src.clone()
    want[13:20] = patch.cpu()
    assert torch.equal(dst.cpu(), want)
    with pytest.raises(ops.KernelError, match="pinned"):
        ops.table_load(torch.zeros(1000, dtype=torch.int32), dst)
    with pytest.raises(ops.KernelError, match="does not fit"):
        ops.table_load(src, dst, patch, 995)


def test_sampler_top_k_one_is_greedy_and_frequencies(ops):
    V = 50
    logits = torch.randn(1, V, generator=torch.Generator().manual_seed(4))
    n = 4000
    rows = logits.expand(n, V).contiguous().to(DEV)
    u = torch.rand(n, generator=torch.Generator().manual_seed(5))
    out = torch.empty(n, dtype=torch.int32, device=DEV)
    ones = torch.ones(n)
    ops.sample(rows, (ones * 0.9).to(DEV), torch.ones(n, dtype=torch.int32).to(DEV), ones.to(DEV), u.to(DEV), out)
    assert set(out.cpu().tolist()) == {int(logits.argmax())}
    ops.sample(rows, (ones * 0.9).to(DEV), torch.full((n,), -1, dtype=torch.int32).to(DEV), ones.to(DEV), u.to(DEV), out)
    freq = torch.bincount(out.cpu().long(), minlength=V).double() / n
    probs = torch.softmax(logits[0].double() / 0.9, 0)
    assert (freq - probs).abs().max() < 0.03
