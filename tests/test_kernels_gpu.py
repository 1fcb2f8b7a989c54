"""Each HIP kernel alone against a plain torch float32/float64 reference of the same
operation, at sizes other than the engine's tiny models (widths and vocabularies that
are no power of two, grouped heads, odd page sizes)."""

import math

import numpy as np
import pytest
import torch

from torch_ops import TorchOps, plain_sample

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module")
def ops():
    from distie_amd.kernels.hip_ops import HipOps

    return HipOps("cuda:0")


def rand(*shape, dtype=torch.float32, seed=0, scale=1.0):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return (torch.randn(*shape, generator=g, device="cuda") * scale).to(dtype)


def close(got, want, dtype, scale=1.0):
    tol = 2e-5 if dtype == torch.float32 else 1.0 / 128
    err = (got.double() - want.double()).abs().max().item()
    assert err <= tol * scale, f"max error {err} > {tol * scale}"


@pytest.mark.parametrize("dtype", DTYPES)
def test_embed(ops, dtype):
    table = rand(301, 72, dtype=dtype)
    ids = torch.tensor([0, 300, 5, 5, 17], dtype=torch.int32, device="cuda")
    got = ops.embed(ids, table)
    assert got.dtype == torch.float32
    assert torch.equal(got, table[ids.long()].float())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,width", [(7, 40), (7, 1000), (7, 1002), (7, 3000), (7, 5000), (7, 8200),
                                        (2100, 1536), (5000, 332), (9000, 64)])     # many rows: two groups a thread
def test_rmsnorm_and_fused_add(ops, dtype, rows, width):
    x = rand(rows, width, seed=1, scale=3.0)
    w = rand(width, dtype=dtype, seed=2)
    eps = 1e-5
    want = x.double() * torch.rsqrt(x.double().pow(2).mean(-1, keepdim=True) + eps) * w.double()
    got = ops.dense(ops.rmsnorm(x, w, eps, dtype))          # (few rows in bfloat16 are normed when they are read)
    assert got.dtype == dtype
    close(got, want, dtype, scale=want.abs().max().item())
    delta = rand(rows, width, dtype=dtype, seed=3)
    res = x.clone()
    got = ops.dense(ops.add_rmsnorm(res, delta, w, eps, dtype))
    s = x.double() + delta.double()
    assert torch.allclose(res.double(), s, atol=1e-6)
    want = s * torch.rsqrt(s.pow(2).mean(-1, keepdim=True) + eps) * w.double()
    close(got, want, dtype, scale=want.abs().max().item())


@pytest.mark.parametrize("width,slices", [(1536, 14), (1536, 4), (96, 9), (4100, 3), (250, 5), (8192, 17)])
def test_add_rmsnorm_adds_slices_in_order(ops, width, slices):
    from distie_amd.kernels.hip_ops import PartialSums

    rows = 5
    res = rand(rows, width, seed=1, scale=2.0)
    part = rand(slices, rows, width, seed=2)
    w = rand(width, dtype=torch.bfloat16, seed=3)
    total = part[0].clone()
    for s in range(1, slices):
        total += part[s]                       # float32, in order, as the kernel
    want_res = res + total
    want = want_res.double() * torch.rsqrt(want_res.double().pow(2).mean(-1, keepdim=True) + 1e-6) * w.double()
    got = ops.add_rmsnorm(res, PartialSums(part, torch.bfloat16), w, 1e-6, torch.bfloat16)
    assert torch.equal(res, want_res)
    close(got, want, torch.bfloat16, scale=want.abs().max().item())


@pytest.mark.parametrize("xd,wd", [(torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16),
                                   (torch.bfloat16, torch.float32), (torch.float32, torch.bfloat16)])
@pytest.mark.parametrize("M,N,K", [(1, 100, 72), (5, 333, 250), (70, 65, 129), (200, 130, 64)])
def test_gemm_generic(ops, xd, wd, M, N, K):
    x, w, b = rand(M, K, dtype=xd, seed=1), rand(N, K, dtype=wd, seed=2), rand(N, seed=3)
    want = x.double() @ w.double().T + b.double()
    got = ops._linear(x, w, b, xd) if not (xd == wd == torch.bfloat16) else None
    if got is None:
        # bf16 x bf16 goes to the matrix-core kernels; call the generic kernel directly
        got = torch.empty(M, N, dtype=xd, device="cuda")
        assert ops._ops.distie_gemm_generic(x.data_ptr(), 1, w.data_ptr(), 1, b.data_ptr(), got.data_ptr(), 1,
                                            M, N, K, None) == 0
    close(got, want, xd, scale=want.abs().max().item())
    got32 = ops.linear_f32out(x, w) if not (xd == wd == torch.bfloat16) else None
    if got32 is not None:
        assert got32.dtype == torch.float32
        close(got32, x.double() @ w.double().T, torch.float32, scale=want.abs().max().item())


@pytest.mark.parametrize("xd,wd", [(torch.float32, torch.float32), (torch.bfloat16, torch.float32),
                                   (torch.float32, torch.bfloat16)])
@pytest.mark.parametrize("M", [1, 2, 3, 5, 8, 9, 17, 64, 65])
@pytest.mark.parametrize("N,K", [(100, 72), (333, 256), (1536, 8960), (7, 8), (2050, 1536)])
def test_products_of_few_rows_in_float32_stream_the_weights(ops, xd, wd, M, N, K):
    """Up to 64 rows in float32 (or against a weight that is kept in float32) go through the kernel that streams
    the weights and multiplies on the vector ALU: the same values as the tiled float32 kernel within float32
    rounding (another order of the sums), whatever the row count, with and without a bias."""
    x, w, b = rand(M, K, dtype=xd, seed=1), rand(N, K, dtype=wd, seed=2), rand(N, seed=3)
    want = x.double() @ w.double().T + b.double()
    scale = want.abs().max().item()
    got = ops._linear(x, w, b, xd)
    assert got.dtype == xd and tuple(got.shape) == (M, N)
    close(got, want, xd, scale=scale)
    tiled = torch.empty(M, N, dtype=xd, device="cuda")
    code = {torch.float32: 0, torch.bfloat16: 1}
    assert ops._ops.distie_gemm_generic(x.data_ptr(), code[xd], w.data_ptr(), code[wd], b.data_ptr(), tiled.data_ptr(),
                                        code[xd], M, N, K, None) == 0
    assert (got.float() - tiled.float()).abs().max().item() <= (2e-5 if xd == torch.float32 else 2 ** -7) * scale
    logits = ops.linear_f32out(x, w)
    assert logits.dtype == torch.float32
    close(logits, x.double() @ w.double().T, torch.float32, scale=scale)
    if M <= 64:
        # it is this kernel that ran: its entry point gives the same bits
        direct = torch.empty(M, N, dtype=torch.float32, device="cuda")
        assert ops._ops.distie_gemv_rows(x.data_ptr(), code[xd], w.data_ptr(), code[wd], None, direct.data_ptr(), 0,
                                         M, N, K, None) == 0
        assert torch.equal(direct, logits)
    assert ops._ops.distie_gemv_rows(x.data_ptr(), code[xd], w.data_ptr(), code[wd], None, logits.data_ptr(), 0,
                                     65, N, K, None) == -1                     # more rows than it takes: refused


@pytest.mark.parametrize("M", [1, 3, 16, 17, 33, 64])
@pytest.mark.parametrize("N,K", [(48, 128), (100, 264), (1536, 1536), (333, 8960), (2050, 72)])
def test_gemm_skinny_bf16(ops, M, N, K):
    x, w, b = rand(M, K, dtype=torch.bfloat16, seed=1), rand(N, K, dtype=torch.bfloat16, seed=2), rand(N, seed=3)
    want = x.double() @ w.double().T
    got = ops.linear_f32out(x, w)
    close(got, want, torch.float32, scale=5 * want.abs().max().item())
    got = ops.dense(ops.linear(x, w, b))
    assert got.dtype == torch.bfloat16
    close(got, want + b.double(), torch.bfloat16, scale=want.abs().max().item())


@pytest.mark.parametrize("M", [1, 3, 8, 16, 17, 33, 50, 64, 65, 96, 130, 192])
@pytest.mark.parametrize("N,K", [(48, 128), (100, 264), (1536, 1536), (333, 8960), (2050, 72), (16, 8), (7, 40)])
def test_gemm_packed_bf16(ops, M, N, K):
    """The same products through the weight's packed copy (what `prepare_linear` leaves): rows and
    k that do not fill a tile, one slice and several, with and without a bias."""
    from distie_amd.kernels.hip_ops import PartialSums, PendingProduct

    x, w, b = rand(M, K, dtype=torch.bfloat16, seed=1), rand(N, K, dtype=torch.bfloat16, seed=2), rand(N, seed=3)
    natural = ops.dense(ops.linear(x, w, b)).float()
    ops.prepare_linear(w)
    assert w._distie_packed.numel() == -(-N // 16) * -(-K // 32) * 512
    want = x.double() @ w.double().T
    got = ops.linear_f32out(x, w)
    close(got, want, torch.float32, scale=5 * want.abs().max().item())
    # 17 to 64 rows: small weights go through the one-wave kernel once per 16 rows, large ones through
    # the kernel that shares x in LDS; both are run for every shape
    # (and that one takes more than 32 rows in one pass or in two, by the weight's size)
    routes = [(ops.ROW_GROUPS_MAX_ELEMENTS, ops.TWO_PASS_MAX_ELEMENTS)] if M <= 16 else [(0, 0), (0, 1 << 40), (1 << 40, 0)]
    try:
        for limit, two_pass in routes:
            ops.ROW_GROUPS_MAX_ELEMENTS, ops.TWO_PASS_MAX_ELEMENTS = limit, two_pass
            part = ops.linear(x, w, b)
            if M <= 16:
                # few rows: the product waits for its reader (the residual sum takes it in; see the test of
                # the decode products); any other reader sees it through `dense`, computed the usual way
                assert isinstance(part, PendingProduct)
            elif limit > 0:
                assert isinstance(part, PartialSums) == (K >= 768)
            got = ops.dense(part)
            assert got.dtype == torch.bfloat16
            close(got, want + b.double(), torch.bfloat16, scale=want.abs().max().item())
            # the packed and the natural kernel add the same products in another order: float32 rounding only
            assert (got.float() - natural).abs().max().item() <= 2 ** -7 * want.abs().max().item()
    finally:
        del ops.ROW_GROUPS_MAX_ELEMENTS, ops.TWO_PASS_MAX_ELEMENTS
    assert ops.ROW_GROUPS_MAX_ELEMENTS == type(ops).ROW_GROUPS_MAX_ELEMENTS


def test_fewer_rows_through_the_packed_kernels_in_a_captured_step(ops):
    """Launched kernel by kernel, a step of up to 192 tokens is bound by the host and takes the packed
    kernels with their fused epilogues; in a captured step only up to 96 rows do, the library's products
    being faster on the device beyond."""
    from distie_amd.kernels.hip_ops import PartialSums

    x, w = rand(120, 1536, dtype=torch.bfloat16, seed=1), rand(64, 1536, dtype=torch.bfloat16, seed=2)
    ops.prepare_linear(w)
    want = x.double() @ w.double().T
    assert not ops.captured
    eager = ops.linear(x, w)
    assert isinstance(eager, PartialSums)
    ops.captured = True
    try:
        captured = ops.linear(x, w)
        assert isinstance(ops.linear(x[:90], w), PartialSums)
    finally:
        ops.captured = False
    assert not isinstance(captured, PartialSums)
    close(ops.dense(eager), want, torch.bfloat16, scale=want.abs().max().item())
    close(captured, want, torch.bfloat16, scale=want.abs().max().item())
    # a weight too large for the memory-side cache to hold between the passes keeps them in a captured step too
    more = rand(150, 1536, dtype=torch.bfloat16, seed=3)
    assert isinstance(ops.linear(more, w), PartialSums)
    ops.PACKED_LARGE_ELEMENTS = 0                   # every weight counts as large
    ops.captured = True
    try:
        large = ops.linear(more, w)
        assert isinstance(large, PartialSums)
        assert not isinstance(ops.linear(rand(200, 1536, dtype=torch.bfloat16, seed=4), w), PartialSums)
    finally:
        ops.captured = False
        del ops.PACKED_LARGE_ELEMENTS
    close(ops.dense(large), more.double() @ w.double().T, torch.bfloat16, scale=want.abs().max().item())
    # ... if its K is longer than it has rows; a large weight with more rows than K leaves after one pass of up to 96
    # rows of x, and after 64 once the library's kernels were timed for that many rows
    wide, x96 = rand(3072, 1536, dtype=torch.bfloat16, seed=5), rand(96, 1536, dtype=torch.bfloat16, seed=6)
    ops.prepare_linear(wide)
    ops.PACKED_LARGE_ELEMENTS = 0
    try:
        one_pass = ops.linear(x96, wide)
        assert isinstance(one_pass, PartialSums) and not isinstance(ops.linear(x[:100], wide), PartialSums)
        ops.library_timed_rows = 192
        through_library = ops.linear(x96, wide)
        assert not isinstance(through_library, PartialSums) and isinstance(ops.linear(x96[:64], wide), PartialSums)
    finally:
        ops.library_timed_rows = 0
        del ops.PACKED_LARGE_ELEMENTS
    want = x96.double() @ wide.double().T
    close(ops.dense(one_pass), want, torch.bfloat16, scale=want.abs().max().item())
    close(through_library, want, torch.bfloat16, scale=want.abs().max().item())


@pytest.mark.parametrize("M", [1, 5, 16, 17, 40, 64, 81, 96, 150, 192])
@pytest.mark.parametrize("I,K", [(88, 2048), (8, 32), (172, 64), (250, 96), (4484, 1536), (13, 72)])
def test_linear_silu_mul_fused(ops, M, I, K):
    x = rand(M, K, dtype=torch.bfloat16, seed=1)
    w = rand(2 * I, K, dtype=torch.bfloat16, seed=5, scale=2.0 / K ** 0.5)
    gu = x.double() @ w.double().T
    want = gu[:, :I] / (1 + torch.exp(-gu[:, :I])) * gu[:, I:]
    # unfused, a product that is not cut along K is rounded to bfloat16 before the activation: gate, up
    # and result each carry a rounding (2^-8 of the value at most), where the fused kernel rounds once
    unfused = ops.linear_silu_mul(x, w)
    close(unfused, want, torch.bfloat16, scale=2 * want.abs().max().item())
    ops.prepare_linear(w, gated=True)
    assert w._distie_gated.numel() == -(-I // 8) * -(-K // 32) * 512
    for two_pass in (1 << 40, 0):           # more than 32 rows in two passes over the weight, or in one
        ops.TWO_PASS_MAX_ELEMENTS = two_pass
        try:
            got = ops.linear_silu_mul(x, w)
        finally:
            del ops.TWO_PASS_MAX_ELEMENTS
        assert got.dtype == torch.bfloat16 and tuple(got.shape) == (M, I)
        close(got, want, torch.bfloat16, scale=want.abs().max().item())
    # more rows than the fused kernel takes: the unfused path, same result
    big = rand(230, K, dtype=torch.bfloat16, seed=2)
    gu = big.double() @ w.double().T
    want = gu[:, :I] / (1 + torch.exp(-gu[:, :I])) * gu[:, I:]
    close(ops.linear_silu_mul(big, w), want, torch.bfloat16, scale=2 * want.abs().max().item())


@pytest.mark.parametrize("M", [1, 5, 16, 17, 45, 64, 70, 96, 129, 224])
@pytest.mark.parametrize("heads,kv_heads,dim,K,P", [(3, 1, 32, 2048, 4), (12, 2, 128, 1536, 16), (4, 4, 16, 72, 16),
                                                    (5, 5, 48, 240, 8), (2, 1, 80, 520, 16), (7, 1, 256, 136, 32),
                                                    (28, 4, 128, 3584, 16), (10, 2, 64, 5000, 16), (20, 4, 48, 3200, 8)])
@pytest.mark.parametrize("with_bias,write", [(True, True), (False, True), (True, False)])
def test_linear_rope_kv_write_fused(ops, M, heads, kv_heads, dim, K, P, with_bias, write):
    """The q/k/v product with rotation and cache write in its epilogue, against product, rotation
    and write one after the other in plain torch. The last three weights are large enough for the wide kernel:
    from 49 rows on the product runs there, on the same copy of the weight (rotation partners side by side, the
    sums written to the columns the rows have in the weight itself), and rotation and write follow as a kernel
    of their own that adds the slices of K."""
    N = (heads + 2 * kv_heads) * dim
    x = rand(M, K, dtype=torch.bfloat16, seed=1)
    w = rand(N, K, dtype=torch.bfloat16, seed=6, scale=1.0 / K ** 0.5)
    b = rand(N, seed=7) if with_bias else None
    pages = 2 * M + 2
    g = torch.Generator().manual_seed(M * 131 + dim)
    slots = torch.randperm(pages * P, generator=g)[:M].tolist()
    positions = torch.randint(0, 5000, (M,), generator=g).tolist()
    meta = make_meta(positions, list(range(M)), list(range(M + 1)), [p + 1 for p in positions],
                     [[0] * 8] * M, slots, P)
    inv_freq = (1.0 / (10000.0 ** (torch.arange(0, dim, 2, dtype=torch.float32) / dim))).cuda()
    k1 = rand(pages, kv_heads, P, dim, dtype=torch.bfloat16, seed=8)
    v1 = rand(pages, kv_heads, dim, P, dtype=torch.bfloat16, seed=9)
    k2, v2 = k1.clone(), v1.clone()
    dense = x.double() @ w.double().T + (b.double() if with_bias else 0.0)
    want = TorchOps("cuda").rope_kv_write(dense.float().clone(), meta, 0, k2, v2, inv_freq, heads, kv_heads, dim, write)
    ops.prepare_linear(w, rotary=(heads, kv_heads, dim))
    assert hasattr(w, "_distie_rotary")
    got = ops.linear_rope_kv_write(x, w, b, meta, 0, k1, v1, inv_freq, heads, kv_heads, dim, write)
    assert got.dtype == torch.bfloat16 and tuple(got.shape) == (M, N)
    scale = want.abs().max().item()
    close(got, want, torch.bfloat16, scale=scale)
    # the cache: the new tokens' places hold what the result holds, every other place is untouched
    close(k1, k2, torch.bfloat16, scale=scale)
    close(v1, v2, torch.bfloat16, scale=scale)
    untouched = torch.ones(pages * P, dtype=torch.bool)
    if write:
        untouched[slots] = False
    keep = untouched.view(pages, P).cuda()
    assert torch.equal(k1.permute(0, 2, 1, 3)[keep], k2.permute(0, 2, 1, 3)[keep])
    assert torch.equal(v1.permute(0, 3, 1, 2)[keep], v2.permute(0, 3, 1, 2)[keep])
    if write:
        view = got.view(M, heads + 2 * kv_heads, dim)
        at = torch.tensor(slots).cuda()
        assert torch.equal(k1[at // P, :, at % P], view[:, heads:heads + kv_heads])
        assert torch.equal(v1[at // P, :, :, at % P], view[:, heads + kv_heads:])
    if M > 64 and N * K > ops.ROW_GROUPS_MAX_ELEMENTS:
        # a weight that the memory-side cache cannot hold between passes is taken in passes of up to 96 rows
        k4, v4 = k2.clone(), v2.clone()
        if write:
            k4[at // P, :, at % P] = 0
        ops.TWO_PASS_MAX_ELEMENTS = 0
        try:
            again = ops.linear_rope_kv_write(x, w, b, meta, 0, k4, v4, inv_freq, heads, kv_heads, dim, write)
        finally:
            del ops.TWO_PASS_MAX_ELEMENTS
        assert torch.equal(again, got) and torch.equal(k4, k1) and torch.equal(v4, v1)
    # unfused (no packed copy), the same within rounding
    w2 = w.clone()
    k3, v3 = k2.clone(), v2.clone()
    unfused = ops.linear_rope_kv_write(x, w2, b, meta, 0, k3, v3, inv_freq, heads, kv_heads, dim, write)
    close(unfused, want, torch.bfloat16, scale=2 * scale)


@pytest.mark.parametrize("M", [1, 5, 8, 9, 16])
@pytest.mark.parametrize("C,I,heads,kv_heads,dim", [(1536, 4484, 12, 2, 128), (72, 13, 3, 1, 16), (3584, 300, 4, 4, 48),
                                                    (4096, 88, 2, 1, 80), (264, 172, 5, 5, 32)])
def test_decode_products_with_the_norm_in_front_and_the_residual_sum_behind(ops, M, C, I, heads, kv_heads, dim):
    """Steps of few rows: a product that is added to the residual stream adds itself (nothing is handed on as
    partial sums), the norm of the stream is left to the product that reads it, and that product computes it
    in front of its own work: gate+up with the activation, q/k/v with bias, rotation and cache write, and the
    head in float32. Each against the same operations one after the other."""
    from distie_amd.kernels.hip_ops import KernelError, PendingNorm, PendingProduct

    eps = 1e-5
    # the product that feeds the stream: y [M, C] = a [M, I] W^T + b, added to the residual in place
    a = rand(M, I * 8, dtype=torch.bfloat16, seed=1)
    w_out = rand(C, I * 8, dtype=torch.bfloat16, seed=2, scale=1.0 / (I * 8) ** 0.5)
    b_out = rand(C, seed=3)
    ops.prepare_linear(w_out)
    residual = rand(M, C, seed=4)
    want_residual = residual.double() + a.double() @ w_out.double().T + b_out.double()
    g = (1 + 0.2 * rand(C, seed=5)).to(torch.bfloat16)
    delta = ops.linear(a, w_out, b_out)
    assert isinstance(delta, PendingProduct) and tuple(delta.shape) == (M, C)
    normed = ops.add_rmsnorm(residual, delta, g, eps, torch.bfloat16)
    scale = want_residual.abs().max().item()
    assert (residual.double() - want_residual).abs().max().item() <= 2e-5 * max(1.0, scale) * 8
    assert isinstance(normed, PendingNorm) and tuple(normed.shape) == (M, C)
    want_normed = want_residual * torch.rsqrt(want_residual.pow(2).mean(-1, keepdim=True) + eps) * g.double()
    xn = ops.dense(normed)
    assert xn.dtype == torch.bfloat16
    close(xn, want_normed, torch.bfloat16, scale=want_normed.abs().max().item())
    xn = xn.double()                       # what the products below see: the norm rounded to bfloat16
    # gate + up with the activation
    w_gu = rand(2 * I, C, dtype=torch.bfloat16, seed=6, scale=2.0 / C ** 0.5)
    ops.prepare_linear(w_gu, gated=True)
    gu = xn @ w_gu.double().T
    want = gu[:, :I] / (1 + torch.exp(-gu[:, :I])) * gu[:, I:]
    got = ops.linear_silu_mul(normed, w_gu)
    assert got.dtype == torch.bfloat16 and tuple(got.shape) == (M, I)
    close(got, want, torch.bfloat16, scale=1.5 * want.abs().max().item())
    # q/k/v with bias, rotation and cache write
    P = 16
    N = (heads + 2 * kv_heads) * dim
    w_qkv = rand(N, C, dtype=torch.bfloat16, seed=7, scale=1.0 / C ** 0.5)
    b_qkv = rand(N, seed=8)
    ops.prepare_linear(w_qkv, rotary=(heads, kv_heads, dim))
    pages = 2 * M + 2
    gen = torch.Generator().manual_seed(M * 17 + dim)
    slots = torch.randperm(pages * P, generator=gen)[:M].tolist()
    positions = torch.randint(0, 5000, (M,), generator=gen).tolist()
    meta = make_meta(positions, list(range(M)), list(range(M + 1)), [p + 1 for p in positions], [[0] * 8] * M, slots, P)
    inv_freq = (1.0 / (10000.0 ** (torch.arange(0, dim, 2, dtype=torch.float32) / dim))).cuda()
    k1 = rand(pages, kv_heads, P, dim, dtype=torch.bfloat16, seed=9)
    v1 = rand(pages, kv_heads, dim, P, dtype=torch.bfloat16, seed=10)
    k2, v2 = k1.clone(), v1.clone()
    dense = (xn @ w_qkv.double().T + b_qkv.double()).float()
    want = TorchOps("cuda").rope_kv_write(dense.clone(), meta, 0, k2, v2, inv_freq, heads, kv_heads, dim, True)
    got = ops.linear_rope_kv_write(normed, w_qkv, b_qkv, meta, 0, k1, v1, inv_freq, heads, kv_heads, dim, True)
    assert got.dtype == torch.bfloat16 and tuple(got.shape) == (M, N)
    close(got, want, torch.bfloat16, scale=1.5 * want.abs().max().item())
    close(k1, k2, torch.bfloat16, scale=1.5 * want.abs().max().item())
    close(v1, v2, torch.bfloat16, scale=1.5 * want.abs().max().item())
    at = torch.tensor(slots).cuda()
    view = got.view(M, heads + 2 * kv_heads, dim)
    assert torch.equal(k1[at // P, :, at % P], view[:, heads:heads + kv_heads])
    assert torch.equal(v1[at // P, :, :, at % P], view[:, heads + kv_heads:])
    # the head: float32 logits
    V = 1001
    w_head = rand(V, C, dtype=torch.bfloat16, seed=11, scale=1.0 / C ** 0.5)
    ops.prepare_linear(w_head)
    logits = ops.linear_f32out(normed, w_head)
    assert logits.dtype == torch.float32 and tuple(logits.shape) == (M, V)
    want = xn @ w_head.double().T
    assert (logits.double() - want).abs().max().item() <= 2e-3 * want.abs().max().item()
    # a norm that was left for later is of no use once its stream has moved on
    ops.add_rmsnorm(residual, ops.linear(a, w_out, b_out), g, eps, torch.bfloat16)
    with pytest.raises(KernelError, match="had changed"):
        ops.linear_silu_mul(normed, w_gu)
    # rows that the fused products do not take are normed at once
    wide = rand(3, 4100, seed=12)
    assert isinstance(ops.rmsnorm(wide, rand(4100, seed=13), eps, torch.bfloat16), torch.Tensor)
    assert isinstance(ops.rmsnorm(rand(17, C, seed=14), g, eps, torch.bfloat16), torch.Tensor)


def test_partial_sums_are_added_by_their_readers(ops):
    """A product over a long K comes back as slices; norm, activation and rotation add them."""
    from distie_amd.kernels.hip_ops import PartialSums

    M, K = 5, 2048
    x = rand(M, K, dtype=torch.bfloat16, seed=1)
    # residual add + norm
    w = rand(96, K, dtype=torch.bfloat16, seed=2, scale=0.05)
    part = ops.linear(x, w)
    assert isinstance(part, PartialSums) and part.slices > 1
    delta = x.double() @ w.double().T
    res = rand(M, 96, seed=3)
    want_res = res.double() + delta
    g = rand(96, dtype=torch.bfloat16, seed=4)
    got = ops.add_rmsnorm(res, part, g, 1e-6, torch.bfloat16)
    assert torch.allclose(res.double(), want_res, atol=1e-4)
    want = want_res * torch.rsqrt(want_res.pow(2).mean(-1, keepdim=True) + 1e-6) * g.double()
    close(got, want, torch.bfloat16, scale=want.abs().max().item())
    # gated activation
    w = rand(2 * 88, K, dtype=torch.bfloat16, seed=5, scale=0.05)
    part = ops.linear(x, w)
    assert isinstance(part, PartialSums)
    gu = x.double() @ w.double().T
    want = gu[:, :88] / (1 + torch.exp(-gu[:, :88])) * gu[:, 88:]
    close(ops.silu_mul(part), want, torch.bfloat16, scale=want.abs().max().item())
    # rotation + cache write, with a bias
    heads, kv_heads, dim, P = 3, 1, 32, 4
    w = rand((heads + 2 * kv_heads) * dim, K, dtype=torch.bfloat16, seed=6, scale=0.05)
    b = rand((heads + 2 * kv_heads) * dim, seed=7)
    part = ops.linear(x, w, b)
    assert isinstance(part, PartialSums)
    dense = (x.double() @ w.double().T + b.double()).float()
    meta = make_meta([7, 8, 9, 0, 30], [0, 0, 0, 1, 2], [0, 3, 4, 5], [10, 1, 31], [[2, 0, 1, -1, -1, -1, -1, -1]] * 3,
                     [0 * P + 3, 1 * P + 0, 1 * P + 1, 5 * P, 6 * P + 2], P)
    inv_freq = (1.0 / (10000.0 ** (torch.arange(0, dim, 2, dtype=torch.float32) / dim))).cuda()
    k1 = torch.zeros(8, kv_heads, P, dim, dtype=torch.bfloat16, device="cuda")
    v1 = torch.zeros(8, kv_heads, dim, P, dtype=torch.bfloat16, device="cuda")
    k2, v2 = torch.zeros_like(k1), torch.zeros_like(v1)
    got = ops.rope_kv_write(part, meta, 0, k1, v1, inv_freq, heads, kv_heads, dim, True)
    want = TorchOps("cuda").rope_kv_write(dense.clone(), meta, 0, k2, v2, inv_freq, heads, kv_heads, dim, True)
    assert got.dtype == torch.bfloat16
    close(got, want, torch.bfloat16, scale=want.abs().max().item())
    close(k1, k2, torch.bfloat16, scale=want.abs().max().item())
    close(v1, v2, torch.bfloat16, scale=want.abs().max().item())
    # any other reader sees the finished sum
    close(ops.dense(part), dense, torch.bfloat16, scale=dense.abs().max().item())


def test_packed_copies_are_left_out_when_memory_is_short(ops, monkeypatch, caplog):
    """A packed copy that would leave less than PACKED_KEEPS_FREE of the device's memory free is not made; the
    product then streams the stored layout and gives the same result."""
    import logging

    x, w = rand(8, 264, dtype=torch.bfloat16, seed=1), rand(1000, 264, dtype=torch.bfloat16, seed=2)
    want = x.double() @ w.double().T
    free, total = torch.cuda.mem_get_info()
    monkeypatch.setattr(torch.cuda, "mem_get_info", lambda *a: (int(0.3 * total) + 1000, total))
    left_out = ops._packed_left_out
    with caplog.at_level(logging.WARNING, logger="distie_amd.kernels.hip_ops"):
        ops.prepare_linear(w, role="down")
    assert not hasattr(w, "_distie_packed") and ops._packed_left_out == left_out + 1
    assert left_out > 0 or "left out" in caplog.text
    close(ops.dense(ops.linear(x, w)), want, torch.bfloat16, scale=want.abs().max().item())
    monkeypatch.undo()
    ops.prepare_linear(w, role="down")
    assert hasattr(w, "_distie_packed")
    close(ops.dense(ops.linear(x, w)), want, torch.bfloat16, scale=want.abs().max().item())


def test_gemm_large_bf16_uses_library_and_matches(ops):
    x, w, b = rand(300, 136, dtype=torch.bfloat16, seed=1), rand(250, 136, dtype=torch.bfloat16, seed=2), rand(250, seed=3)
    want = x.double() @ w.double().T + b.double()
    before = ops.library_plans()[0]
    close(ops.linear(x, w, b), want, torch.bfloat16, scale=want.abs().max().item())
    close(ops.linear(x, w), want - b.double(), torch.bfloat16, scale=want.abs().max().item())
    assert ops.library_plans()[0] == before + 2          # with and without bias: two plans, made once
    close(ops.linear(x, w, b), want, torch.bfloat16, scale=want.abs().max().item())
    assert ops.library_plans()[0] == before + 2
    # the head's product: float32 out, unrounded sums
    logits = ops.linear_f32out(x, w)
    assert logits.dtype == torch.float32
    close(logits, want - b.double(), torch.float32, scale=want.abs().max().item())


def test_library_kernels_chosen_by_timing(ops):
    """With tuning on, a new shape has the library's candidates timed once; the result is the same product."""
    x, w = rand(512, 264, dtype=torch.bfloat16, seed=4), rand(384, 264, dtype=torch.bfloat16, seed=5)
    want = x.double() @ w.double().T
    timed = ops.library_plans()[1]
    ops.tune_library_products(True)
    try:
        got = ops.linear(x, w)
    finally:
        ops.tune_library_products(False)
    assert ops.library_plans()[1] == timed + 1
    close(got, want, torch.bfloat16, scale=want.abs().max().item())
    close(ops.linear(x, w), want, torch.bfloat16, scale=want.abs().max().item())
    assert ops.library_plans()[1] == timed + 1


@pytest.mark.parametrize("M,N,K", [(300, 250, 136), (2048, 1536, 1024), (65, 1000, 333)])
def test_gemm_large_float32_is_a_float32_product(ops, M, N, K):
    """Large float32 products go to the library's float32 kernels: every product and sum in float32. An error
    bound far below what a product of operands cut to 10 or 7 bits of mantissa would leave (a relative 5e-4 and
    4e-3 per product) pins that no reduced-precision mode is in use; with a bias, with tuning, and with a K that
    is no multiple of 8."""
    x, w, b = rand(M, K, seed=1), rand(N, K, seed=2), rand(N, seed=3)
    want = x.double() @ w.double().T
    scale = (x.double().abs() @ w.double().abs().T).max().item()       # what the rounding errors scale with
    before = ops.library_plans()[0]
    got = ops.linear(x, w)
    assert got.dtype == torch.float32 and ops.library_plans()[0] == before + 1
    assert (got.double() - want).abs().max().item() < 3e-6 * scale
    got = ops.linear(x, w, b)
    assert (got.double() - want - b.double()).abs().max().item() < 3e-6 * scale
    ops.tune_library_products(True)
    try:
        tuned = ops.linear(x, w)
    finally:
        ops.tune_library_products(False)
    assert (tuned.double() - want).abs().max().item() < 3e-6 * scale
    assert (ops.linear_f32out(x, w).double() - want).abs().max().item() < 3e-6 * scale


@pytest.mark.parametrize("bias", [False, True])
def test_gemm_large_bf16_with_a_ragged_last_round(ops, bias, monkeypatch):
    """A large product whose columns end a little after a whole round of the library's tiles is run as two
    products into one output; with a tile of 16 (patched) a small case takes that path. The result is the
    plain product's."""
    monkeypatch.setattr(type(ops), "LIBRARY_TILE", 16)
    M = 600
    round_columns = ops._compute_units // -(-M // 16) * 16
    N = 2 * round_columns + 24
    assert ops._library_tail(M, N) == 24 and ops._library_tail(M, 2 * round_columns) == 0
    assert ops._library_tail(M, round_columns + round_columns // 2) == 0        # many columns left: one product
    x, w = rand(M, 136, dtype=torch.bfloat16, seed=1), rand(N, 136, dtype=torch.bfloat16, seed=2)
    b = rand(N, seed=3) if bias else None
    want = x.double() @ w.double().T + (b.double() if bias else 0)
    got = ops.linear(x, w, b)
    assert got.shape == (M, N) and got.is_contiguous()
    close(got, want, torch.bfloat16, scale=want.abs().max().item())


def make_meta(positions, token_request, cu_q, kv_len, tables, slots, block_size):
    from distie_amd.kernels.interface import BatchMeta, GroupMeta

    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device="cuda")
    B = len(kv_len)
    return BatchMeta(num_tokens=len(positions), num_requests=B, positions=i32(positions),
                     token_request=i32(token_request), cu_q=i32(cu_q), kv_len=i32(kv_len),
                     state_slots=i32([0] * B), max_q=max(b - a for a, b in zip(cu_q, cu_q[1:])),
                     max_kv=max(kv_len), block_size=block_size,
                     groups=[GroupMeta(block_table=i32(tables), slots=i32(slots))],
                     host_cu_q=np.asarray(cu_q), all_decode=all(b - a == 1 for a, b in zip(cu_q, cu_q[1:])))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,dim,pairs", [(4, 2, 16, 8), (3, 1, 32, 16), (5, 5, 48, 24), (12, 2, 128, 64), (2, 2, 64, 16)])
def test_rope_kv_write(ops, dtype, heads, kv_heads, dim, pairs):
    P, pages = 4, 9
    positions = [0, 1, 2, 3, 4, 100, 7]
    token_request = [0, 0, 0, 0, 0, 1, 2]
    slots = [3 * P + 0, 3 * P + 1, 3 * P + 2, 3 * P + 3, 0 * P + 0, 7 * P + 0, 5 * P + 3]
    meta = make_meta(positions, token_request, [0, 5, 6, 7], [5, 101, 8], [[3, 0, -1]] * 3, slots, P)
    qkv = rand(7, (heads + 2 * kv_heads) * dim, dtype=dtype, seed=4)
    inv_freq = (1.0 / (10000.0 ** (torch.arange(0, 2 * pairs, 2, dtype=torch.float32) / (2 * pairs)))).cuda()
    k1 = torch.zeros(pages, kv_heads, P, dim, dtype=dtype, device="cuda")
    v1 = torch.zeros(pages, kv_heads, dim, P, dtype=dtype, device="cuda")
    k2, v2, qkv2 = k1.clone(), v1.clone(), qkv.clone()
    ops.rope_kv_write(qkv, meta, 0, k1, v1, inv_freq, heads, kv_heads, dim, True)
    ref = TorchOps("cuda")
    ref.rope_kv_write(qkv2, meta, 0, k2, v2, inv_freq, heads, kv_heads, dim, True)
    close(qkv, qkv2, dtype, scale=4.0)
    close(k1, k2, dtype, scale=4.0)
    assert torch.equal(v1, v2)
    # float64 check of the rotation at a far position, where the angle's rounding matters
    view = qkv.view(7, heads + 2 * kv_heads, dim)
    src = qkv2.new_tensor(rand(7, (heads + 2 * kv_heads) * dim, dtype=dtype, seed=4).double().cpu().numpy()).view(7, -1, dim)
    ang = torch.tensor(100.0, dtype=torch.float32) * inv_freq.cpu()   # float32 angle, as specified
    a, b = src[5, 0, :pairs].double().cpu(), src[5, 0, pairs:2 * pairs].double().cpu()
    want = torch.cat([a * ang.double().cos() - b * ang.double().sin(), b * ang.double().cos() + a * ang.double().sin()])
    close(view[5, 0, :2 * pairs].cpu(), want, dtype, scale=4.0)
    if 2 * pairs < dim:
        assert torch.equal(view[5, 0, 2 * pairs:], src[5, 0, 2 * pairs:].to(dtype).cuda())
    # without writing, the cache stays as it is
    k3 = torch.zeros_like(k1)
    ops.rope_kv_write(qkv.clone(), meta, 0, k3, torch.zeros_like(v1), inv_freq, heads, kv_heads, dim, False)
    assert k3.abs().sum() == 0


@pytest.mark.parametrize("P", [16, 32, 24, 8])
@pytest.mark.parametrize("heads,kv_heads,dim", [(12, 2, 128), (3, 1, 48), (4, 4, 16)])
def test_rope_kv_write_of_long_portions(ops, heads, kv_heads, dim, P):
    """bfloat16 portions of many tokens: 16 tokens in a row that lie inside one page have their values written
    as one run (pages of 16 and 32; a page of 24 holds such a run only where it starts at a multiple of 8 and
    ends inside the page; a page of 8 never), the others value by value: a request that starts at a page's first
    place, one that starts in the middle of a page (its groups of 16 straddle pages), one of 5 tokens, one
    whose pages lie in falling order. Values equal bit for bit, keys and q within rounding; what no token owns
    stays as it was."""
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(P + dim)
    starts, counts = [0, 2 * P + 5, 7, 3 * P], [70, 45, 5, 64]
    pages_needed = sum(-(-(a + n) // P) for a, n in zip(starts, counts))
    order = torch.randperm(pages_needed + 2, generator=g).tolist()
    positions, token_request, slots, cu_q, tables, lens = [], [], [], [0], [], []
    for b, (a, n) in enumerate(zip(starts, counts)):
        mine = sorted((order.pop() for _ in range(-(-(a + n) // P))), reverse=b == 3)
        tables.append(mine)
        for pos in range(a, a + n):
            positions.append(pos)
            token_request.append(b)
            slots.append(mine[pos // P] * P + pos % P)
        cu_q.append(len(positions))
        lens.append(a + n)
    width = max(len(t) for t in tables)
    tables = [t + [-1] * (width - len(t)) for t in tables]
    meta = make_meta(positions, token_request, cu_q, lens, tables, slots, P)
    T = len(positions)
    qkv = rand(T, (heads + 2 * kv_heads) * dim, dtype=dtype, seed=6)
    inv_freq = (1.0 / (10000.0 ** (torch.arange(0, dim, 2, dtype=torch.float32) / dim))).cuda()
    k1 = rand(pages_needed + 2, kv_heads, P, dim, dtype=dtype, seed=7)
    v1 = rand(pages_needed + 2, kv_heads, dim, P, dtype=dtype, seed=8)
    k2, v2, qkv2 = k1.clone(), v1.clone(), qkv.clone()
    got = ops.rope_kv_write(qkv, meta, 0, k1, v1, inv_freq, heads, kv_heads, dim, True)
    want = TorchOps("cuda").rope_kv_write(qkv2, meta, 0, k2, v2, inv_freq, heads, kv_heads, dim, True)
    close(got, want, dtype, scale=4.0)
    close(k1, k2, dtype, scale=4.0)
    assert torch.equal(v1, v2)
    # into a cache of zeros: only the places the tokens own are written
    k3, v3 = k2.clone().zero_(), v2.clone().zero_()
    # (the kernel surface rotates in place; the library itself also writes to another buffer, which the test
    # double cannot ask for: here the input is a fresh copy and the cache starts from zeros)
    again = ops.rope_kv_write(rand(T, (heads + 2 * kv_heads) * dim, dtype=dtype, seed=6), meta, 0, k3, v3, inv_freq, heads,
                              kv_heads, dim, True)
    held = torch.zeros_like(v3, dtype=torch.bool)
    for slot in slots:
        held[slot // P, :, :, slot % P] = True
    assert torch.equal(v3[held], v2[held]) and v3[~held].abs().sum() == 0
    close(again, want, dtype, scale=4.0)


def paged_case(heads, kv_heads, dim, P, lens, q_lens, dtype, seed=0):
    """Requests with `lens` cached tokens (the last `q_lens` of them new), pages in a shuffled order."""
    g = torch.Generator().manual_seed(seed)
    total_pages = sum(-(-n // P) for n in lens) + 3
    order = torch.randperm(total_pages, generator=g).tolist()
    width = max(-(-n // P) for n in lens) + 1
    tables, positions, token_request, cu_q, slots = [], [], [], [0], []
    for b, (n, q) in enumerate(zip(lens, q_lens)):
        pages = [order.pop() for _ in range(-(-n // P))]
        tables.append(pages + [-1] * (width - len(pages)))
        for pos in range(n - q, n):
            positions.append(pos)
            token_request.append(b)
            slots.append(pages[pos // P] * P + pos % P)
        cu_q.append(len(positions))
    meta = make_meta(positions, token_request, cu_q, lens, tables, slots, P)
    k = rand(total_pages, kv_heads, P, dim, dtype=dtype, seed=seed + 1)
    v = rand(total_pages, kv_heads, dim, P, dtype=dtype, seed=seed + 2)
    qkv = rand(len(positions), (heads + 2 * kv_heads) * dim, dtype=dtype, seed=seed + 3)
    return meta, qkv, k, v


ATTENTION_SHAPES = [
    (4, 2, 16, 4, None), (3, 1, 32, 8, 8), (5, 5, 48, 16, 20), (12, 2, 128, 16, None),
    (6, 3, 64, 5, 33), (8, 1, 80, 16, None), (2, 2, 256, 32, 100), (4, 2, 16, 16, 7), (40, 2, 32, 16, None),
    (12, 2, 128, 64, 150), (4, 2, 64, 16, 1000),
    (3, 1, 40, 16, None), (2, 2, 40, 8, 9)]        # a head size that is no multiple of 16: the wave-per-token kernel


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,dim,P,window", ATTENTION_SHAPES)
def test_paged_attention(ops, dtype, heads, kv_heads, dim, P, window):
    """Mixed step: whole prompts, portions down to two tokens, single decoded tokens."""
    lens, q_lens = [70, 1, 33, 130, 200, 67], [70, 1, 2, 1, 17, 66]
    meta, qkv, k, v = paged_case(heads, kv_heads, dim, P, lens, q_lens, dtype)
    got = ops.paged_attention(qkv, meta, 0, k, v, heads, kv_heads, dim, dim ** -0.5, window)
    want = TorchOps("cuda").paged_attention(qkv.double(), meta, 0, k.double(), v.double(), heads, kv_heads, dim,
                                            dim ** -0.5, window)
    close(got, want, dtype, scale=want.abs().max().item())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,dim,P,window", [(4, 2, 16, 16, None), (3, 1, 48, 16, 100), (12, 2, 128, 16, None),
                                                         (2, 1, 256, 32, 300), (6, 2, 64, 64, 70)])
def test_paged_attention_long_portions(ops, dtype, heads, kv_heads, dim, P, window):
    """Portions that span several tiles of queries and of keys, with and without a past; and the
    tiled kernel taking the single tokens too."""
    lens, q_lens = [520, 260, 131, 400], [300, 260, 1, 129]
    meta, qkv, k, v = paged_case(heads, kv_heads, dim, P, lens, q_lens, dtype, seed=3)
    want = TorchOps("cuda").paged_attention(qkv.double(), meta, 0, k.double(), v.double(), heads, kv_heads, dim,
                                            dim ** -0.5, window)
    got = ops.paged_attention(qkv, meta, 0, k, v, heads, kv_heads, dim, dim ** -0.5, window)
    close(got, want, dtype, scale=want.abs().max().item())
    meta.host_cu_q = None
    got = ops.paged_attention(qkv, meta, 0, k, v, heads, kv_heads, dim, dim ** -0.5, window)
    close(got, want, dtype, scale=want.abs().max().item())


@pytest.mark.parametrize("heads,kv_heads,dim,P,window", [(4, 2, 16, 16, None), (12, 2, 128, 16, None), (3, 1, 48, 16, 700),
                                                         (2, 1, 256, 32, 100), (6, 2, 64, 64, None)])
@pytest.mark.parametrize("parts", [2, 3, 5, 8, 16])
@pytest.mark.parametrize("dtype", DTYPES)
def test_paged_attention_keys_walked_in_parts(ops, dtype, heads, kv_heads, dim, P, window, parts, monkeypatch):
    """From 1,024 visible keys on, the tiled kernel cuts the walk over the keys into parts and merges: a long
    portion without a past, one that starts in the middle of a tile after a long past, a short one, a
    two-token one, and single tokens (which the decode kernel takes, or the tiled kernel too). In float32 the
    tiled float32 kernel takes the whole step where the head size allows it."""
    lens, q_lens = [1300, 1500, 90, 777, 40, 1100], [1300, 100, 90, 1, 2, 1]
    meta, qkv, k, v = paged_case(heads, kv_heads, dim, P, lens, q_lens, dtype, seed=5)
    monkeypatch.setattr(type(ops), "PREFILL_PARTS", ((64, parts),))      # as a longer context would have it
    want = TorchOps("cuda").paged_attention(qkv.double(), meta, 0, k.double(), v.double(), heads, kv_heads, dim,
                                            dim ** -0.5, window)
    got = ops.paged_attention(qkv, meta, 0, k, v, heads, kv_heads, dim, dim ** -0.5, window)
    close(got, want, dtype, scale=want.abs().max().item())
    # The merge reads only what the kernel before it wrote in this call: whatever the buffers between the two
    # kernels held before (here: NaN everywhere), the result is the same.
    filled = 0
    for plan in meta.scratch.values():
        for name in ("prefill_o", "prefill_ml"):
            if isinstance(plan, dict) and name in plan:
                plan[name].fill_(float("nan"))
                filled += 1
    tiled = dtype == torch.bfloat16 or (dim % 32 == 0 and dim <= 128)       # else: the wave-per-token kernel, no parts
    assert (filled >= 2) == tiled
    again = ops.paged_attention(qkv, meta, 0, k, v, heads, kv_heads, dim, dim ** -0.5, window)
    assert torch.equal(again, got)
    meta.host_cu_q = None                      # the tiled kernel takes the single tokens too
    got = ops.paged_attention(qkv, meta, 0, k, v, heads, kv_heads, dim, dim ** -0.5, window)
    close(got, want, dtype, scale=want.abs().max().item())
    # in one walk, the same within rounding
    monkeypatch.setattr(type(ops), "PREFILL_PARTS", ())
    whole = ops.paged_attention(qkv, meta, 0, k, v, heads, kv_heads, dim, dim ** -0.5, window)
    close(whole, want, dtype, scale=want.abs().max().item())


@pytest.mark.parametrize("requests,heads,kv_heads,dim,P", [(65, 8, 4, 64, 16), (100, 28, 4, 128, 16), (200, 12, 2, 128, 32),
                                                           (150, 4, 4, 48, 16), (700, 3, 1, 32, 16), (80, 10, 5, 80, 64)])
def test_decode_steps_of_many_requests_share_one_run_length(ops, monkeypatch, requests, heads, kv_heads, dim, P):
    """Where cutting every request into the same number of runs would leave a fifth of the waves unused (here:
    wherever no window applies), the requests of a decode step share one run length, found on the device from the
    step's lengths: requests of 1 to
    1,500 keys (a long one gets several runs, a short one a single one, some end on a run's edge), then one far
    longer than the others (it is what bounds the run length), then all of one length; as launched for these
    lengths and as in a captured step that was made for far longer ones. Against plain attention."""
    import random

    monkeypatch.setattr(type(ops), "DECODE_SHARED_BELOW", 1.01)
    rng = random.Random(requests)
    for lens in ([rng.choice([1, 2, 63, 64, 65, 128, 640, 1280]) if i % 3 == 0 else rng.randint(1, 1500) for i in range(requests)],
                 [4000] + [rng.randint(1, 90) for _ in range(requests - 1)],
                 [333] * requests):
        meta, qkv, k, v = paged_case(heads, kv_heads, dim, P, lens, [1] * requests, torch.bfloat16, seed=requests)
        assert meta.all_decode
        want = TorchOps("cuda").paged_attention(qkv.double(), meta, 0, k.double(), v.double(), heads, kv_heads, dim,
                                                dim ** -0.5, None)
        for limit in (max(lens), 8192):
            meta.max_kv = limit
            meta.scratch.clear()
            got = ops.paged_attention(qkv, meta, 0, k, v, heads, kv_heads, dim, dim ** -0.5, None)
            plans = [plan for plan in meta.scratch.values() if isinstance(plan, dict) and "run_len" in plan]
            assert len(plans) == 1 and plans[0]["run_len"] is not None, "the step did not take the shared run length"
            run_len = int(plans[0]["run_len"].item())
            budget, most = ops.DECODE_WAVES // kv_heads, plans[0]["max_splits"]
            runs = lambda length: sum(-(-n // length) for n in lens)
            assert run_len % 64 == 0 and max(-(-n // run_len) for n in lens) <= most
            # the shortest that keeps the runs within the waves, unless the longest request asks for a longer one
            assert runs(run_len) <= budget or run_len >= -(-max(lens) // 64) * 64
            assert run_len == 64 or runs(run_len - 64) > budget or -(-max(lens) // (run_len - 64)) > most
            close(got, want, torch.bfloat16, scale=want.abs().max().item())
        # under a window, or with fewer requests, every request is cut by its own length as before
        windowed = ops.paged_attention(qkv, meta, 0, k, v, heads, kv_heads, dim, dim ** -0.5, 100)
        assert all(plan.get("run_len") is None for key, plan in meta.scratch.items() if isinstance(plan, dict) and key[1] == 100)
        want = TorchOps("cuda").paged_attention(qkv.double(), meta, 0, k.double(), v.double(), heads, kv_heads, dim,
                                                dim ** -0.5, 100)
        close(windowed, want, torch.bfloat16, scale=want.abs().max().item())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,dim,P,window", ATTENTION_SHAPES)
def test_paged_attention_decode_step(ops, dtype, heads, kv_heads, dim, P, window):
    """Every request brings one token (the split-key kernel in bfloat16), contexts from 1 to 1,100 (the last:
    under a window of 100 its first visible key lies in the second half of a run of 64)."""
    lens = [1, 2, 16, 17, 64, 65, 129, 300, 700, 1100]
    meta, qkv, k, v = paged_case(heads, kv_heads, dim, P, lens, [1] * len(lens), dtype)
    assert meta.all_decode
    want = TorchOps("cuda").paged_attention(qkv.double(), meta, 0, k.double(), v.double(), heads, kv_heads, dim,
                                            dim ** -0.5, window)
    got = ops.paged_attention(qkv, meta, 0, k, v, heads, kv_heads, dim, dim ** -0.5, window)
    close(got, want, dtype, scale=want.abs().max().item())
    # as in a captured step: the launch is sized for the longest context the model allows (more places for
    # partial results than any of these requests fills, and a wrong guess of where their runs begin)
    for limit in (4096, 20000):
        meta.max_kv = limit
        got = ops.paged_attention(qkv, meta, 0, k, v, heads, kv_heads, dim, dim ** -0.5, window)
        close(got, want, dtype, scale=want.abs().max().item())
    # two requests, one of them long: more runs than the quick combination of partial results takes, while
    # the short request fills two of its places
    meta, qkv, k, v = paged_case(heads, kv_heads, dim, P, [5000, 70], [1, 1], dtype, seed=3)
    want = TorchOps("cuda").paged_attention(qkv.double(), meta, 0, k.double(), v.double(), heads, kv_heads, dim,
                                            dim ** -0.5, window)
    for limit in (5000, 32768):
        meta.max_kv = limit
        got = ops.paged_attention(qkv, meta, 0, k, v, heads, kv_heads, dim, dim ** -0.5, window)
        close(got, want, dtype, scale=want.abs().max().item())


@pytest.mark.parametrize("heads,kv_heads,dim,P", [(12, 2, 128, 16), (4, 2, 64, 16), (3, 1, 48, 16), (2, 1, 256, 32)])
@pytest.mark.parametrize("per_key", [0.1, 1.0, -0.1, 0.02])
@pytest.mark.parametrize("dtype", DTYPES)
def test_prefill_attention_scores_that_grow_along_the_keys(ops, dtype, heads, kv_heads, dim, P, per_key):
    """The tiled kernel lets a column's reference score lag behind its largest score by up to a factor of 2^8
    in weight before it scales the sums down. Scores that rise by `per_key` (in units of log 2) from one key
    to the next cross that bound every few tiles of 64 keys (0.1), every tile (1.0), never after the first
    (falling scores) or once in a long while (0.02); a portion without a past and one behind 500 tokens.

    In float32 with scores that double every key, a row's largest score s (up to 620, from products near
    7,000) is known to float32 only to s * 2^-23 a rounding, so its weights are known to that relative error
    and no kernel can do better: each row is held to the usual bound plus four such roundings of its own
    largest score (rows near the start of a sequence to the usual bound alone, rows at 900 keys to 3e-4 of
    the largest value; a sum scaled wrongly by 2^8 is off by the value itself)."""
    lens, q_lens = [700, 900], [700, 400]
    meta, qkv, k, v = paged_case(heads, kv_heads, dim, P, lens, q_lens, dtype, seed=11)
    scale = dim ** -0.5
    q = qkv.view(qkv.shape[0], heads + 2 * kv_heads, dim)
    q[:, :heads, 0] = 8.0
    slope = per_key / (8.0 * scale * 1.4426950408889634)
    for b, n in enumerate(lens):
        for pos in range(n):
            page = int(meta.groups[0].block_table[b, pos // P])
            k[page, :, pos % P, 0] = slope * pos
    want = TorchOps("cuda").paged_attention(qkv.double(), meta, 0, k.double(), v.double(), heads, kv_heads, dim, scale, None)
    got = ops.paged_attention(qkv, meta, 0, k, v, heads, kv_heads, dim, scale, None)
    if dtype == torch.float32 and per_key == 1.0:
        size = want.abs().max().item()
        largest_score = per_key / 1.4426950408889634 * meta.positions.double() + 8.0      # of each row: its last key's, and the rest of the product
        allowed = 2e-5 * size + 4 * largest_score * 2.0 ** -23 * size
        err = (got.double() - want.double()).abs().amax(dim=1)
        assert bool((err <= allowed).all()), f"row {int((err - allowed).argmax())}: {err.max().item()}"
        assert allowed.min().item() < 3e-5 * size and allowed.max().item() < 4e-4 * size
        return
    close(got, want, dtype, scale=want.abs().max().item())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,dim,P,window", [(4, 2, 16, 4, None), (12, 2, 128, 16, None), (3, 1, 40, 16, 9), (6, 3, 64, 5, 33)])
def test_paged_attention_with_slopes_and_a_cap(ops, dtype, heads, kv_heads, dim, P, window):
    """What a variant of attention adds to the scores (`ScoreExtras`): the matrix-core kernels compute plain
    attention, so such a step goes to the wave-per-token kernel, in both precisions; slopes of the wrong shape
    are refused."""
    from distie_amd.kernels.hip_ops import KernelError
    from distie_amd.kernels.interface import ScoreExtras

    lens, q_lens = [70, 1, 33, 130, 200, 67], [70, 1, 2, 1, 17, 66]
    meta, qkv, k, v = paged_case(heads, kv_heads, dim, P, lens, q_lens, dtype)
    slopes = torch.tensor([0.5 ** (h + 1) for h in range(heads)], device="cuda")
    plain_out = ops.paged_attention(qkv, meta, 0, k, v, heads, kv_heads, dim, dim ** -0.5, window)
    for extras in (ScoreExtras(head_slopes=slopes), ScoreExtras(score_cap=2.0), ScoreExtras(slopes, 1.5)):
        got = ops.paged_attention(qkv, meta, 0, k, v, heads, kv_heads, dim, dim ** -0.5, window, extras)
        want = TorchOps("cuda").paged_attention(qkv.double(), meta, 0, k.double(), v.double(), heads, kv_heads, dim,
                                                dim ** -0.5, window, extras)
        close(got, want, dtype, scale=want.abs().max().item())
        assert (got.float() - plain_out.float()).abs().max().item() > 0.05
    same = ops.paged_attention(qkv, meta, 0, k, v, heads, kv_heads, dim, dim ** -0.5, window, ScoreExtras())
    assert torch.equal(same, plain_out)                       # nothing set: plain attention, the same kernels
    with pytest.raises(KernelError, match="head_slopes"):
        ops.paged_attention(qkv, meta, 0, k, v, heads, kv_heads, dim, dim ** -0.5, window, ScoreExtras(slopes[:-1]))
    with pytest.raises(ValueError):
        ScoreExtras(score_cap=0.0)


def test_a_norm_left_for_later_notices_that_its_residual_changed(ops):
    """Few rows in bfloat16: `rmsnorm` hands out a value that the next product computes. If the residual is
    written in between (by torch, also through a view, or by a kernel here) the value is refused."""
    from distie_amd.kernels.hip_ops import KernelError, PendingNorm

    w = rand(64, dtype=torch.bfloat16, seed=1)
    weight = rand(48, 64, dtype=torch.bfloat16, seed=2)
    ops.prepare_linear(weight)
    for change in (lambda x: x.add_(1.0), lambda x: x[:2].mul_(2.0), lambda x: x.view(-1)[3:5].zero_(),
                   lambda x: ops.add_rmsnorm(x, torch.ones_like(x), w, 1e-6, torch.bfloat16)):
        x = rand(4, 64, seed=3)
        normed = ops.rmsnorm(x, w, 1e-6, torch.bfloat16)
        assert isinstance(normed, PendingNorm)
        ops.dense(normed)                                     # unchanged: fine, as often as asked
        change(x)
        with pytest.raises(KernelError, match="changed"):
            ops.linear(normed, weight)
        with pytest.raises(KernelError, match="ops.dense"):
            normed.float()
    x = rand(4, 64, seed=3)
    want = ops.dense(ops.linear(ops.dense(ops.rmsnorm(x, w, 1e-6, torch.bfloat16)), weight))
    got = ops.dense(ops.linear(ops.rmsnorm(x, w, 1e-6, torch.bfloat16), weight))
    close(got, want, torch.bfloat16, scale=want.abs().max().item())


def test_attention_takes_a_positive_scale_only(ops):
    from distie_amd.kernels.hip_ops import KernelError

    meta, qkv, k, v = paged_case(4, 2, 32, 16, [40], [40], torch.bfloat16, seed=2)
    for scale in (0.0, -0.1, float("nan")):
        with pytest.raises(KernelError, match="scale"):
            ops.paged_attention(qkv, meta, 0, k, v, 4, 2, 32, scale, None)


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_finds_one_far_key(ops, dtype):
    """One key among hundreds gets a large score: the output must be that key's value,
    wherever the key sits (first of a page, last of a page, the window's edge)."""
    heads, kv_heads, dim, P = 4, 2, 32, 16
    for far, window in [(0, None), (15, None), (16, None), (287, None), (300 - 64, 64), (299, 64)]:
        meta, qkv, k, v = paged_case(heads, kv_heads, dim, P, [300], [1], dtype, seed=5)
        q = qkv.view(1, heads + 2 * kv_heads, dim)
        page = int(meta.groups[0].block_table[0, far // P])
        k[page, :, far % P] = 0
        k[page, :, far % P, 0] = 30.0
        q[0, :heads] = 0
        q[0, :heads, 0] = 30.0
        want = v[page, :, :, far % P].float().repeat_interleave(2, dim=0).reshape(1, -1)
        for decode in (False, True):
            meta.all_decode = decode
            meta.host_cu_q = np.asarray([0, 1]) if decode else None      # None: the tiled kernel takes the single token
            got = ops.paged_attention(qkv, meta, 0, k, v, heads, kv_heads, dim, dim ** -0.5, window)
            close(got, want, dtype, scale=4.0)
    # just outside the window the key must not count
    meta, qkv, k, v = paged_case(heads, kv_heads, dim, P, [300], [1], dtype, seed=5)
    far = 299 - 64
    page = int(meta.groups[0].block_table[0, far // P])
    k[page, :, far % P, 0] = 1000.0
    qkv.view(1, -1, dim)[0, :heads, 0] = 30.0
    got = ops.paged_attention(qkv, meta, 0, k, v, heads, kv_heads, dim, dim ** -0.5, 64)
    want = TorchOps("cuda").paged_attention(qkv.double(), meta, 0, k.double(), v.double(), heads, kv_heads, dim,
                                            dim ** -0.5, 64)
    close(got, want, dtype, scale=4.0)


@pytest.mark.parametrize("dtype", DTYPES)
def test_silu_mul_and_gather(ops, dtype):
    gu = rand(9, 2 * 173, dtype=dtype, seed=6, scale=3.0)
    g, u = gu[:, :173].double(), gu[:, 173:].double()
    want = g / (1 + torch.exp(-g)) * u
    close(ops.silu_mul(gu), want, dtype, scale=want.abs().max().item())
    x = rand(11, 77, dtype=dtype, seed=7)
    rows = torch.tensor([10, 0, 3, 3], dtype=torch.int32, device="cuda")
    assert torch.equal(ops.gather_rows(x, rows), x[rows.long()])


def test_upload_of_small_host_arrays(ops):
    """More uploads in a row than there are staging buffers, of several types and sizes (one beyond a
    buffer's first size): each arrives as it was, whatever was uploaded after it."""
    rng = np.random.default_rng(0)
    sent = []
    for i in range(3 * ops.UPLOAD_BUFFERS + 1):
        dtype = (np.int32, np.int64, np.float32)[i % 3]
        n = (1, 7, 64, 3000)[i % 4]
        values = (rng.standard_normal(n) * 1000).astype(dtype)
        sent.append((values, ops.upload(values)))
    sent.append((np.zeros((0,), np.int32), ops.upload(np.zeros((0,), np.int32))))
    sent.append((np.arange(12, dtype=np.int64).reshape(3, 4), ops.upload(np.arange(12, dtype=np.int64).reshape(3, 4))))
    for values, dev in sent:
        assert dev.device.type == "cuda" and tuple(dev.shape) == values.shape
        assert dev.dtype == torch.from_numpy(np.empty(0, values.dtype)).dtype
        assert np.array_equal(dev.cpu().numpy(), values)


def test_argmax_and_sample(ops):
    logits = rand(6, 1001, seed=8, scale=2.0)
    logits[1, 7] = logits[1, 900] = 50.0          # equals: the lowest index wins
    logits[2, 1000] = 60.0
    got = ops.argmax(logits)
    assert got.tolist() == [int(r.argmax()) for r in logits[:1]] + [7, 1000] + [int(r.argmax()) for r in logits[3:]]
    big = rand(3, 151936, seed=9)
    big[1, 151935] = big[1, 70000] = 9.0           # equals in different pieces of the row
    big[2, 4096] = 8.0
    assert ops.argmax(big).tolist() == [int(big[0].argmax()), 70000, 4096]
    big[0, 1001] = big[0, 1002] = big[0, 1003] = 11.0      # equals inside one load of four logits
    assert ops.argmax(big).tolist() == [1001, 70000, 4096]
    # rows that do not begin at a multiple of 16 bytes, and a vocabulary that is no multiple of four: one logit a load
    flat = rand(2 * 151936 + 1, seed=12)
    shifted = flat[1:].view(2, 151936)
    shifted[1, 151935] = shifted[1, 151934] = 7.0
    assert shifted.data_ptr() % 16 != 0 and ops.argmax(shifted).tolist() == [int(shifted[0].argmax()), 151934]
    odd = rand(5, 40001, seed=13)
    odd[3, 40000] = 9.0
    odd[4, 17] = odd[4, 39999] = 9.5
    assert ops.argmax(odd).tolist() == [int(r.argmax()) for r in odd[:3]] + [40000, 17]
    temps = torch.tensor([0.0, 0.7, 1.0, 1.5, 0.3, 2.0], device="cuda")
    hits = 0
    trials = 40
    for n in range(trials):
        seeds = torch.arange(6, device="cuda", dtype=torch.int64) * 1000 + n
        counters = torch.full((6,), n, device="cuda", dtype=torch.int64)
        got = ops.sample(logits, temps, seeds, counters)
        want = plain_sample(logits, temps, seeds, counters)
        assert got[0] == want[0]
        hits += int((got == want.cuda()).sum())
    # the float32 cumulative sum may step over a boundary that float64 does not; that is rare
    assert hits >= 6 * trials - 3
    # large vocabularies are drawn from in pieces: the pick's interval of the cumulative distribution (float64)
    # holds the target within float32 rounding; a stretch without weight as long as a piece changes nothing
    from distie_amd.sampling import uniform_of
    for rows, vocab, scale in ((3, 151936, 1.0), (70, 40001, 4.0), (64, 151936, 6.0), (1, 151936, 3.0)):
        logits = rand(rows, vocab, seed=10 + rows, scale=scale)
        logits[0, 5000:30000] = -float("inf")
        temps = torch.tensor([(0.0, 0.7, 1.0, 1.6)[(i + 1) % 4] for i in range(rows)], device="cuda")
        seeds = torch.arange(rows, device="cuda", dtype=torch.int64) * 77 + 5
        counters = torch.arange(rows, device="cuda", dtype=torch.int64) + 3
        got = ops.sample(logits, temps, seeds, counters).tolist()
        for i, (row, t) in enumerate(zip(logits.double().cpu(), temps.tolist())):
            if t <= 0:
                assert got[i] == int(row.argmax())
                continue
            w = torch.exp((row - row.max()) / t)
            c = torch.cumsum(w, 0) / w.sum()
            u = uniform_of(int(seeds[i]), int(counters[i]))
            below = float(c[got[i] - 1]) if got[i] else 0.0
            assert w[got[i]] > 0 and below - 1e-5 <= u <= float(c[got[i]]) + 1e-5, (rows, vocab, i, got[i])
    # the draws follow the distribution: chi-square-free check on a small vocabulary
    small = torch.tensor([[0.0, 1.0, 2.0, -1.0]], device="cuda").repeat(4000, 1)
    draws = ops.sample(small, torch.ones(4000, device="cuda"), torch.full((4000,), 12345, device="cuda", dtype=torch.int64),
                       torch.arange(4000, device="cuda", dtype=torch.int64))
    freq = torch.bincount(draws.long(), minlength=4).double() / 4000
    assert (freq.cpu() - torch.softmax(small[0].double().cpu(), 0)).abs().max() < 0.03
