"""Each HIP kernel alone against a plain torch reference of the same operation, at sizes other
than the engine tests use (head sizes in steps of 16, odd head counts and groups, widths and a
vocabulary that are no power of two)."""

import math

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

PAGE = 64
DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module")
def K():
    from beholdd.kernels import HipKernels
    return HipKernels("cuda:0")


def dev(t):
    return t.to("cuda:0")


def tol(dtype, f32=2e-5, bf16=1.6e-2):
    return f32 if dtype == torch.float32 else bf16


def rel(got, want):
    got, want = got.double().cpu(), want.double().cpu()
    return float((got - want).abs().max() / want.abs().max().clamp_min(1e-30))


def test_library_is_the_in_tree_one(K):
    assert K.library_path.endswith("libbeholdd_hip.so")
    assert K.page_size == PAGE


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,width,vocab", [(1, 96, 331), (37, 1000, 77), (5, 4096, 513)])
def test_embed(K, dtype, rows, width, vocab):
    g = torch.Generator().manual_seed(rows)
    table = torch.randn(vocab, width, generator=g).to(dtype)
    tokens = torch.randint(0, vocab, (rows,), generator=g, dtype=torch.int32)
    tokens[0], tokens[-1] = vocab - 1, 0
    out = torch.empty(rows, width, dtype=torch.float32, device="cuda:0")
    K.embed(dev(tokens), dev(table), out)
    assert torch.equal(out.cpu(), table[tokens.long()].float())


@pytest.mark.parametrize("out_dtype", DTYPES)
@pytest.mark.parametrize("w_dtype", DTYPES)
@pytest.mark.parametrize("rows,width,eps", [(1, 48, 1e-6), (33, 1000, 1e-5), (4, 5120, 1e-6), (3, 4097, 1e-2),
                                            (300, 1000, 1e-5), (257, 4096, 1e-6), (256, 260, 1e-6), (301, 4098, 1e-6),
                                            (258, 256, 1e-6), (270, 2560, 1e-5), (259, 8192, 1e-6),
                                            # many rows and a width that is a multiple of 4: 16 bytes per load
                                            (100, 5120, 1e-6), (64, 16384, 1e-6), (65, 17408, 1e-6), (80, 12, 1e-5)])
def test_rmsnorm(K, out_dtype, w_dtype, rows, width, eps):
    g = torch.Generator().manual_seed(width)
    x = torch.randn(rows, width, generator=g) * 3 + 0.5
    w = (1 + 0.1 * torch.randn(width, generator=g)).to(w_dtype)
    out = torch.empty(rows, width, dtype=out_dtype, device="cuda:0")
    K.rmsnorm(dev(x), dev(w), eps, out)
    want = x.double() / torch.sqrt((x.double() ** 2).mean(-1, keepdim=True) + eps) * w.double()
    assert rel(out, want) < tol(out_dtype, 2e-6, 4e-3)
    # gathered rows, no weight
    index = torch.tensor([rows - 1, 0, rows - 1], dtype=torch.int32)
    out2 = torch.empty(3, width, dtype=out_dtype, device="cuda:0")
    K.rmsnorm(dev(x), None, eps, out2, rows=dev(index))
    want2 = (x.double() / torch.sqrt((x.double() ** 2).mean(-1, keepdim=True) + eps))[index.long()]
    assert rel(out2, want2) < tol(out_dtype, 2e-6, 4e-3)
    if rows >= 64:      # many gathered rows, with a weight
        index = torch.randint(0, rows, (rows + 5,), generator=g, dtype=torch.int32)
        out3 = torch.empty(rows + 5, width, dtype=out_dtype, device="cuda:0")
        K.rmsnorm(dev(x), dev(w), eps, out3, rows=dev(index))
        assert rel(out3, want[index.long()]) < tol(out_dtype, 2e-6, 4e-3)


@pytest.mark.parametrize("a_dtype,w_dtype", [(torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16),
                                             (torch.bfloat16, torch.float32)])
@pytest.mark.parametrize("m,n,k", [(1, 96, 120), (7, 331, 200), (64, 130, 72), (65, 257, 1000), (200, 64, 48),
                                   (3, 1000, 4096), (130, 520, 264), (17, 40, 100), (33, 100, 2048), (48, 16, 8),
                                   (8, 4096, 12288), (300, 1000, 1024), (1, 15, 64),
                                   (1030, 43700, 136)])      # the last: enough tiles for the largest tile shape
def test_gemm(K, a_dtype, w_dtype, m, n, k):
    g = torch.Generator().manual_seed(m * 1000 + n)
    a = torch.randn(m, k, generator=g).to(a_dtype)
    w = (torch.randn(n, k, generator=g) * 0.05).to(w_dtype)
    want = a.double() @ w.double().t()
    f32_bound = 4 * math.sqrt(k) * 2.0 ** -24      # float32 accumulation of k products, a few standard deviations
    for out_dtype in (torch.float32, a_dtype):
        out = torch.empty(m, n, dtype=out_dtype, device="cuda:0")
        K.gemm(dev(a), dev(w), out)
        assert rel(out, want) < tol(out_dtype, f32_bound, 4e-3), (out_dtype, rel(out, want))
    base = torch.randn(m, n, generator=g)
    acc = dev(base.clone())
    K.gemm(dev(a), dev(w), acc, accumulate=True)
    assert rel(acc, want + base.double()) < f32_bound


@pytest.mark.parametrize("m,n,k", [(1, 96, 128), (8, 331, 192), (64, 130, 64), (65, 257, 1024), (200, 64, 448),
                                   (3, 1000, 4096), (130, 520, 256), (16, 24, 64), (33, 16, 2048),
                                   (8, 4096, 12288), (300, 1000, 1024), (129, 129, 128),
                                   (1030, 43700, 192),
                                   # whole tiles of the packed layout (N a multiple of 16), last tiles moved back inside
                                   (300, 1008, 1024), (129, 144, 128), (128, 128, 64), (1030, 43712, 192),
                                   (2048, 4096, 512),
                                   # few whole tiles: K in parts (equal and unequal ones) and a finishing kernel
                                   (200, 320, 832), (512, 4096, 4096), (128, 128, 4096),
                                   # many rows but few of the widest tiles: K in two or four parts of the kernel whose wave groups take turns
                                   (1800, 4096, 2048), (1000, 4096, 4096), (600, 6144, 4096), (760, 6032, 1024),
                                   # 65 to 127 rows: whole tiles of 64 rows
                                   (100, 256, 1024), (127, 4096, 512), (65, 128, 64),
                                   # 33 to 64 rows, K from 512: the waves of a workgroup share the activations through LDS;
                                   # a last slice of fewer than 512 k, weight blocks that do not fill the last workgroup
                                   (33, 128, 512), (48, 144, 576), (64, 4096, 4096), (49, 1008, 1088), (40, 6144, 4096),
                                   (64, 4096, 12288), (57, 5120, 5120), (80, 4096, 4096), (128, 6144, 4096), (97, 1008, 1280),
                                   # up to 32 rows, blocks of 16 weight rows between one and two per compute unit: workgroups
                                   # that own 20, 24 or 28 rows (parts of two or three blocks); a last chunk trip that is not whole
                                   (8, 5120, 1024), (1, 5120, 5120), (32, 7168, 512), (17, 6144, 192), (9, 7168, 5120), (3, 5120, 17408),
                                   # 17 to 32 rows and very many outputs (a head over a long vocabulary): the kernel for 33 to 128 rows
                                   (17, 32768, 512), (32, 40016, 768), (24, 32784, 1024), (16, 32768, 512),
                                   # 49 to 96 rows and many times the chip's workgroups in one part: eight waves a workgroup
                                   (64, 65568, 512), (90, 65536, 768), (49, 66000, 512)])
def test_gemm_with_packed_weights(K, m, n, k):
    """The same product from the regrouped (16 x 64 blocks) weight layout."""
    from beholdd.kernels import PackedWeight
    g = torch.Generator().manual_seed(m * 7 + n)
    a = torch.randn(m, k, generator=g).to(torch.bfloat16)
    w = (torch.randn(n, k, generator=g) * 0.05).to(torch.bfloat16)
    packed = K.pack_weight(dev(w))
    assert isinstance(packed, PackedWeight) and packed.shape == (n, k) and packed.data.numel() == -(-n // 16) * 16 * k
    assert not isinstance(K.pack_weight(dev(w[:, :k - 8].contiguous())), PackedWeight)      # width not a multiple of 64
    assert not isinstance(K.pack_weight(dev(w.float())), PackedWeight)
    want = a.double() @ w.double().t()
    f32_bound = 4 * math.sqrt(k) * 2.0 ** -24
    for out_dtype in (torch.float32, torch.bfloat16):
        out = torch.empty(m, n, dtype=out_dtype, device="cuda:0")
        K.gemm(dev(a), packed, out)
        assert rel(out, want) < tol(out_dtype, f32_bound, 4e-3), (out_dtype, rel(out, want))
    base = torch.randn(m, n, generator=g)
    acc = dev(base.clone())
    K.gemm(dev(a), packed, acc, accumulate=True)
    assert rel(acc, want + base.double()) < f32_bound
    # adding into a bfloat16 matrix: where the kernel for many rows would read blocks it does not run (it adds
    # into float32 only), so the product must not be handed blocks
    base16 = base.to(torch.bfloat16)
    acc16 = dev(base16.clone())
    K.gemm(dev(a), packed, acc16, accumulate=True)
    assert rel(acc16, want + base16.double()) < 8e-3


@pytest.mark.parametrize("g_dtype", DTYPES)
@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("m,n,k,n2", [(1, 192, 128, 48), (8, 4096, 256, 1000), (17, 200, 64, 64), (64, 320, 192, 130),
                                      (48, 512, 1024, 256), (64, 4096, 4096, 2048), (33, 1024, 576, 640),
                                      (96, 1024, 1024, 512), (128, 4096, 4096, 2048),
                                      # workgroups that own 20, 24 or 28 weight rows, on both sides of the norm
                                      (8, 5120, 512, 7168), (20, 6144, 256, 5120), (1, 5120, 128, 6144)])
def test_norm_rides_on_the_products_around_it(K, g_dtype, packed, m, n, k, n2):
    """The product that completes the residual prepares the following RMSNorm (rows times the norm weight,
    partial sums of squares), and the product after it applies each row's factor to its result."""
    from beholdd.kernels import NormedRows
    from beholdd.parts.base import NormRequest
    if m > 64 and not packed:
        pytest.skip("beyond 64 rows a norm rides on products of packed weights only")
    gen = torch.Generator().manual_seed(m * 31 + n)
    a = torch.randn(m, k, generator=gen).to(torch.bfloat16)
    w = (torch.randn(n, k, generator=gen) * 0.1).to(torch.bfloat16)
    base = torch.randn(m, n, generator=gen) * 3
    g = (1 + 0.3 * torch.randn(n, generator=gen)).to(g_dtype)
    eps = 1e-5
    residual = dev(base.clone())
    w_dev = K.pack_weight(dev(w)) if packed else dev(w)
    prepared = K.gemm(dev(a), w_dev, residual, accumulate=True, then_norm=NormRequest(dev(g), eps))
    assert isinstance(prepared, NormedRows) and prepared.shape == (m, n)
    want_residual = base.double() + a.double() @ w.double().t()
    assert rel(residual, want_residual) < 4 * math.sqrt(k) * 2.0 ** -24
    got_residual = residual.cpu().double()
    assert rel(prepared.rows, got_residual * g.double()) < 4e-3                       # bfloat16 rounding
    assert rel(prepared.ss.sum(1), (got_residual ** 2).sum(-1)) < 1e-5
    assert prepared.ss.shape[0] == m and prepared.ss.dim() == 2
    normed = got_residual / torch.sqrt((got_residual ** 2).mean(-1, keepdim=True) + eps) * g.double()

    w2 = (torch.randn(n2, n, generator=gen) * 0.1).to(torch.bfloat16)
    w2_dev = K.pack_weight(dev(w2)) if packed else dev(w2)
    for out_dtype in (torch.float32, torch.bfloat16):
        out = torch.empty(m, n2, dtype=out_dtype, device="cuda:0")
        assert K.gemm(prepared, w2_dev, out) is None
        assert rel(out, normed @ w2.double().t()) < 8e-3, rel(out, normed @ w2.double().t())
    # a product that cannot take the prepared form runs the norm itself, from the residual
    out = torch.empty(m, n2, dtype=torch.float32, device="cuda:0")
    K.gemm(prepared, dev(w2.float()), out)
    assert rel(out, normed @ w2.double().t()) < 8e-3
    if n2 % 2 == 0:
        half = n2 // 2
        act = torch.empty(m, half, dtype=torch.bfloat16, device="cuda:0")
        K.gemm_swiglu(prepared, w2_dev, act)
        gate, up = normed @ w2[:half].double().t(), normed @ w2[half:].double().t()
        assert rel(act, gate / (1 + torch.exp(-gate)) * up) < 1.2e-2


@pytest.mark.parametrize("m,n,k,n2,g_dtype", [(200, 320, 192, 130, torch.float32), (200, 320, 192, 144, torch.bfloat16),
                                              (128, 128, 64, 128, torch.bfloat16), (256, 4096, 128, 256, torch.float32),
                                              (200, 320, 832, 144, torch.float32), (256, 1024, 512, 1024, torch.bfloat16),
                                              (100, 320, 832, 144, torch.float32), (65, 128, 64, 128, torch.bfloat16),
                                              (200, 320, 832, 25088, torch.float32),
                                              (300, 4096, 128, 256, torch.float32), (3072, 16384, 64, 256, torch.float32)])
def test_norm_rides_on_wide_products(K, m, n, k, n2, g_dtype):
    """The same for products of 65 to 256 rows: whole tiles of a packed weight carry the norm, by themselves
    (partial sums per tile column, edge tiles counting only what they own) or through the kernel that
    finishes the parts of K; other wide products, and those of more rows, leave it alone."""
    from beholdd.kernels import NormedRows
    from beholdd.parts.base import NormRequest
    gen = torch.Generator().manual_seed(m + n)
    a = torch.randn(m, k, generator=gen).to(torch.bfloat16)
    w = (torch.randn(n, k, generator=gen) * 0.1).to(torch.bfloat16)
    base = torch.randn(m, n, generator=gen) * 3
    g = (1 + 0.3 * torch.randn(n, generator=gen)).to(g_dtype)
    eps = 1e-5
    on = lambda t: t.double().to("cuda:0")      # the references of these sizes are computed on the device, by torch
    residual = dev(base.clone())
    assert K.gemm(dev(a), dev(w), residual.clone(), accumulate=True, then_norm=NormRequest(dev(g), eps)) is None
    prepared = K.gemm(dev(a), K.pack_weight(dev(w)), residual, accumulate=True, then_norm=NormRequest(dev(g), eps))
    want_residual = on(base) + on(a) @ on(w).t()
    assert rel(residual, want_residual.cpu()) < 4 * math.sqrt(k) * 2.0 ** -24
    if m > 256:
        assert prepared is None
        return
    assert isinstance(prepared, NormedRows) and prepared.shape == (m, n) and prepared.ss.shape[0] == m
    got_residual = residual.double()
    assert rel(prepared.rows, (got_residual * on(g)).cpu()) < 4e-3
    assert rel(prepared.ss.sum(1), (got_residual ** 2).sum(-1).cpu()) < 1e-5
    normed = got_residual / torch.sqrt((got_residual ** 2).mean(-1, keepdim=True) + eps) * on(g)
    w2 = (torch.randn(n2, n, generator=gen) * 0.1).to(torch.bfloat16)
    want = (normed @ on(w2).t()).cpu()
    for w2_dev in (K.pack_weight(dev(w2)), dev(w2)):        # the second runs the norm itself, from the residual
        for out_dtype in (torch.float32, torch.bfloat16):
            out = torch.empty(m, n2, dtype=out_dtype, device="cuda:0")
            assert K.gemm(prepared, w2_dev, out) is None
            assert rel(out, want) < 8e-3, rel(out, want)
    half = n2 // 2
    act = torch.empty(m, half, dtype=torch.bfloat16, device="cuda:0")
    K.gemm_swiglu(prepared, K.pack_weight(dev(w2)), act)
    gate, up = want[:, :half], want[:, half:]
    assert rel(act, gate / (1 + torch.exp(-gate)) * up) < 1.2e-2


@pytest.mark.parametrize("g_dtype", DTYPES)
@pytest.mark.parametrize("m,n,k", [(2048, 4096, 4096), (1000, 4096, 2048 * 4), (1800, 5120 - 1024, 2048),
                                   (601, 4096, 12288), (2047, 4080, 4096),    # rows and pieces that fill no block
                                   (512, 4096, 4096), (333, 4080, 12288)])    # four parts of the 128-wide tile
def test_product_in_parts_of_many_rows_finishes_the_norm(K, g_dtype, m, n, k):
    """Beyond 256 rows, where K goes through the turns kernel in parts, the finishing kernel owns whole rows and
    writes the norm's output itself: `gemm(..., then_norm=)` returns it as a plain bfloat16 matrix."""
    from beholdd.parts.base import NormRequest
    gen = torch.Generator().manual_seed(m + n)
    a = (torch.randn(m, k, generator=gen) * 0.5).to(torch.bfloat16)
    w = (torch.randn(n, k, generator=gen) * 0.05).to(torch.bfloat16)
    base = torch.randn(m, n, generator=gen) * 3
    g = (1 + 0.3 * torch.randn(n, generator=gen)).to(g_dtype)
    eps = 1e-5
    on = lambda t: t.double().to("cuda:0")
    packed = K.pack_weight(dev(w))
    plain = dev(base.clone())
    assert K.gemm(dev(a), packed, plain, accumulate=True) is None
    residual = dev(base.clone())
    normed = K.gemm(dev(a), packed, residual, accumulate=True, then_norm=NormRequest(dev(g), eps))
    assert isinstance(normed, torch.Tensor) and normed.dtype == torch.bfloat16 and normed.shape == (m, n)
    assert torch.equal(residual, plain)            # the same sums in the same order as without the norm
    assert rel(residual, (on(base) + on(a) @ on(w).t()).cpu()) < 4 * math.sqrt(k) * 2.0 ** -24
    got = residual.double()
    want = got / torch.sqrt((got ** 2).mean(-1, keepdim=True) + eps) * on(g)
    assert rel(normed, want.cpu()) < 4e-3
    reference = torch.empty(m, n, dtype=torch.bfloat16, device="cuda:0")
    K.rmsnorm(residual, dev(g), eps, reference)
    assert (normed.float() - reference.float()).abs().max() <= 2.0 ** -7 * reference.float().abs().max()


def test_norm_does_not_ride_on_wide_steps(K):
    from beholdd.parts.base import NormRequest
    a = torch.randn(65, 64).to(torch.bfloat16)
    w = torch.randn(32, 64).to(torch.bfloat16)
    residual = torch.zeros(65, 32, device="cuda:0")
    assert K.gemm(dev(a), dev(w), residual, accumulate=True, then_norm=NormRequest(dev(torch.ones(32)), 1e-6)) is None
    assert rel(residual, a.double() @ w.double().t()) < 1e-5


@pytest.mark.parametrize("blocks", [8, 6, 4])
@pytest.mark.parametrize("m,n,k", [(256, 256, 128), (300, 400, 384), (520, 1040, 256), (257, 272, 1152),
                                   (1024, 768, 2048), (2400, 1296, 128)])
def test_gemm_whose_wave_groups_take_turns(K, blocks, m, n, k):
    """The product for many rows at each of its tile widths: whole tiles, tiles moved back inside at both
    edges, one and many k steps; float32 with and without accumulation, bfloat16, SwiGLU.  The last size has
    more than eight tiles of rows and a number of weight tiles that is no multiple of four: there the order in
    which the workgroups take the tiles goes in blocks of 8 x 4, with a short block at either edge."""
    g = torch.Generator().manual_seed(m + n + blocks)
    a = torch.randn(m, k, generator=g).to(torch.bfloat16)
    w = (torch.randn(2 * n, k, generator=g) * 0.05).to(torch.bfloat16)
    plain, both = K.pack_weight(dev(w[:n].contiguous())), K.pack_weight(dev(w))
    want = a.double() @ w[:n].double().t()
    f32_bound = 4 * math.sqrt(k) * 2.0 ** -24
    out = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda:0")
    K.gemm_turns(dev(a), plain, out, blocks)
    assert rel(out, want) < f32_bound, rel(out, want)
    base = torch.randn(m, n, generator=g)
    acc = dev(base.clone())
    K.gemm_turns(dev(a), plain, acc, blocks, accumulate=True)
    assert rel(acc, want + base.double()) < f32_bound
    out16 = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda:0")
    K.gemm_turns(dev(a), plain, out16, blocks)
    assert rel(out16, want) < 4e-3, rel(out16, want)
    if n >= 16 * blocks:
        up = a.double() @ w[n:].double().t()
        want_act = want / (1 + torch.exp(-want)) * up
        act = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda:0")
        K.gemm_turns(dev(a), both, act, blocks, swiglu=True)
        assert rel(act, want_act) < 6e-3, rel(act, want_act)


def blocked_reference(x, block_rows=16):
    """x [rows, width] in blocks of 16 (or 8) rows x 32 columns, each block as [4 groups of 8 columns][rows][8],
    the blocks of a group of rows one after the other along the width; rows that x lacks are zero."""
    rows, width = x.shape
    padded = -(-rows // block_rows) * block_rows
    full = torch.zeros(padded, width, dtype=x.dtype)
    full[:rows] = x
    return full.view(padded // block_rows, block_rows, width // 32, 4, 8).permute(0, 2, 3, 1, 4).reshape(-1)


@pytest.mark.parametrize("block_rows", [16, 8])
@pytest.mark.parametrize("rows,width", [(1, 32), (16, 64), (300, 96), (257, 4096), (1000, 160), (5, 4096), (40, 128)])
def test_rows_into_blocks_and_back(K, rows, width, block_rows):
    x = torch.randn(rows, width, generator=torch.Generator().manual_seed(rows)).to(torch.bfloat16)
    blocked = K.to_blocked(dev(x), block_rows=block_rows)
    assert tuple(blocked.shape) == (rows, width) and blocked.block_rows == block_rows
    assert blocked.data.numel() == (-(-rows // 256) * 256 if rows > 32 else -(-rows // block_rows) * block_rows) * width
    want = blocked_reference(x, block_rows)
    assert torch.equal(blocked.data[:want.numel()].cpu(), want)
    assert torch.equal(K.from_blocked(blocked).cpu(), x)
    from beholdd.kernels import KernelError
    with pytest.raises(KernelError, match="multiple of 32"):
        K.to_blocked(dev(torch.zeros(4, 48, dtype=torch.bfloat16)))
    from beholdd.kernels.library import BlockedRows
    short = BlockedRows(torch.zeros(rows * width, dtype=torch.bfloat16, device="cuda:0")[:-1], rows, width, block_rows)
    with pytest.raises(KernelError, match="whole blocks"):      # a buffer that does not hold what the kernels will read
        K.from_blocked(short)


@pytest.mark.parametrize("blocks", [8, 6, 4])
@pytest.mark.parametrize("m,n,k", [(256, 256, 128), (300, 416, 384), (527, 1056, 256), (257, 288, 1152), (1024, 768, 2048),
                                   (2400, 1312, 128)])
def test_gemm_with_turns_reads_and_writes_rows_in_blocks(K, blocks, m, n, k):
    """The same product from activations in blocks of 16 x 32 gives the same bits as from rows (the sums run
    in the same order), also where the last tile of rows sticks out of the matrix and the buffer's rows beyond
    the matrix hold NaN; the gated product writes blocks that hold what it writes as rows."""
    g = torch.Generator().manual_seed(m + n + blocks)
    a = dev(torch.randn(m, k, generator=g).to(torch.bfloat16))
    w = (torch.randn(2 * n, k, generator=g) * 0.05).to(torch.bfloat16)
    plain, both = K.pack_weight(dev(w[:n].contiguous())), K.pack_weight(dev(w))
    from beholdd.kernels.library import BlockedRows
    in_blocks = BlockedRows(torch.full((-(-m // 256) * 256 * k,), float("nan"), dtype=torch.bfloat16, device="cuda:0"), m, k)
    K.to_blocked(a, in_blocks)
    if m % 16:
        assert bool(torch.isnan(in_blocks.data.float()).any())      # the rows of the last tile that do not exist
    for dtype, accumulate in ((torch.float32, False), (torch.float32, True), (torch.bfloat16, False)):
        base = torch.randn(m, n, generator=g).to(dtype)
        from_rows, from_blocks = dev(base.clone()), dev(base.clone())
        K.gemm_turns(a, plain, from_rows, blocks, accumulate=accumulate)
        K.gemm_turns(in_blocks, plain, from_blocks, blocks, accumulate=accumulate)
        assert torch.equal(from_rows, from_blocks)
    if n >= 16 * blocks and n % 32 == 0:
        rows_out = torch.empty(m, n, dtype=torch.bfloat16, device="cuda:0")
        K.gemm_turns(a, both, rows_out, blocks, swiglu=True)
        for source in (a, in_blocks):
            out = BlockedRows(torch.full((-(-m // 256) * 256 * n,), float("nan"), dtype=torch.bfloat16, device="cuda:0"), m, n)
            K.gemm_turns(source, both, out, blocks, swiglu=True)
            assert torch.equal(K.from_blocked(out), rows_out)


@pytest.mark.parametrize("g_dtype", DTYPES)
@pytest.mark.parametrize("m", [1, 2, 3, 8, 9, 16, 17, 32, 33, 48, 64])
def test_products_of_few_rows_hand_each_other_blocks(K, m, g_dtype):
    """A layer's feed-forward and the norms around it as a decode step of m sequences runs them: the norm writes
    its rows for the gated product, that one its output for the down product, which adds into the residual and
    prepares the next norm for the product after it.  Every matrix on the way lies in blocks (of 8 rows up to 8,
    of 16 beyond), as `new_rows` hands them out for their readers; the numbers are those of float64
    within bfloat16's rounding, and matrices handed over as plain rows give the same bits (they are regrouped)."""
    from beholdd.kernels.library import BlockedRows, NormedRows
    from beholdd.parts.base import NormRequest, ProductReader
    hidden, inter = 1024, 1536
    g = torch.Generator().manual_seed(m)
    residual = torch.randn(m, hidden, generator=g)
    w_gate_up = (torch.randn(2 * inter, hidden, generator=g) * 0.05).to(torch.bfloat16)
    w_down = (torch.randn(hidden, inter, generator=g) * 0.05).to(torch.bfloat16)
    g1 = (1 + 0.3 * torch.randn(hidden, generator=g)).to(g_dtype)
    g2 = (1 + 0.3 * torch.randn(hidden, generator=g)).to(g_dtype)
    gate_up, down = K.pack_weight(dev(w_gate_up)), K.pack_weight(dev(w_down))
    eps = 1e-5

    def chain(readers):
        h = dev(residual.clone())
        reader = lambda outputs, swiglu=False: (outputs, swiglu) if readers else ()
        x = K.new_rows(m, hidden, torch.bfloat16, *reader(inter, True))
        K.rmsnorm(h, dev(g1), eps, x)
        act = K.new_rows(m, inter, torch.bfloat16, *reader(hidden))
        K.gemm_swiglu(x, gate_up, act)
        prepared = K.gemm(act, down, h, accumulate=True,
                          then_norm=NormRequest(dev(g2), eps, ProductReader(inter, True) if readers else None))
        assert isinstance(prepared, NormedRows)          # up to 256 rows the norm rides on the products around it
        again = torch.empty(m, inter, dtype=torch.bfloat16, device="cuda:0")
        K.gemm_swiglu(prepared, gate_up, again)
        return h, again, [x, act, prepared.rows]

    h_rows, again_rows, kinds_rows = chain(False)
    h_blocks, again_blocks, kinds_blocks = chain(True)
    assert not any(isinstance(t, BlockedRows) for t in kinds_rows)
    want_blocks = 8 if m <= 8 else 16
    assert [t.block_rows if isinstance(t, BlockedRows) else 0 for t in kinds_blocks] == [want_blocks] * 3
    assert torch.equal(h_rows, h_blocks) and torch.equal(again_rows, again_blocks)
    on = lambda t: t.double().to("cuda:0")
    norm = lambda t, w: t / torch.sqrt((t ** 2).mean(-1, keepdim=True) + eps) * on(w)
    x64 = norm(on(residual), g1).to(torch.bfloat16).double()
    both = x64 @ on(w_gate_up).t()
    act64 = (both[:, :inter] / (1 + torch.exp(-both[:, :inter])) * both[:, inter:]).to(torch.bfloat16).double()
    h64 = on(residual) + act64 @ on(w_down).t()
    assert rel(h_blocks, h64.cpu()) < 3e-3
    both = norm(h64, g2) @ on(w_gate_up).t()
    assert rel(again_blocks, (both[:, :inter] / (1 + torch.exp(-both[:, :inter])) * both[:, inter:]).cpu()) < 2e-2


@pytest.mark.parametrize("m", [300, 1000, 2048])
def test_products_of_many_rows_hand_each_other_blocks(K, m):
    """`new_rows` names the reader: norm -> gated product -> down product with the next norm finished, all through
    rows in blocks, give what the same chain gives through plain matrices."""
    from beholdd.kernels.library import BlockedRows
    from beholdd.parts.base import NormRequest, ProductReader
    hidden, inter = 2048, 8192
    g = torch.Generator().manual_seed(m)
    residual = torch.randn(m, hidden, generator=g)
    gate_up = K.pack_weight(dev((torch.randn(2 * inter, hidden, generator=g) * 0.05).to(torch.bfloat16)))
    down = K.pack_weight(dev((torch.randn(hidden, inter, generator=g) * 0.05).to(torch.bfloat16)))
    g1, g2 = dev(1 + 0.3 * torch.randn(hidden, generator=g)), dev(1 + 0.3 * torch.randn(hidden, generator=g))

    def chain(blocks):
        h = dev(residual.clone())
        reader = lambda outputs, swiglu=False: (outputs, swiglu) if blocks else ()
        x = K.new_rows(m, hidden, torch.bfloat16, *reader(inter, True))
        K.rmsnorm(h, g1, 1e-5, x)
        act = K.new_rows(m, inter, torch.bfloat16, *reader(hidden))
        K.gemm_swiglu(x, gate_up, act)
        normed = K.gemm(act, down, h, accumulate=True,
                        then_norm=NormRequest(g2, 1e-5, ProductReader(inter, True) if blocks else None))
        kinds = [type(x), type(act), type(normed)]
        if normed is None:
            normed = torch.empty(m, hidden, dtype=torch.bfloat16, device="cuda:0")
            K.rmsnorm(h, g2, 1e-5, normed)
        return h, K.from_blocked(normed) if isinstance(normed, BlockedRows) else normed, kinds

    h_rows, normed_rows, kinds_rows = chain(False)
    h_blocks, normed_blocks, kinds_blocks = chain(True)
    assert BlockedRows not in kinds_rows
    if m >= 1000:       # these sizes go to the kernel that reads blocks, and the down product finishes the norm
        assert kinds_blocks == [BlockedRows, BlockedRows, BlockedRows]
    assert torch.equal(h_rows, h_blocks) and torch.equal(normed_rows, normed_blocks)
    assert bool(torch.isfinite(h_blocks).all())


def test_product_of_more_than_two_to_the_31_activation_elements(K):
    """A step of 131,328 rows times 16,384 inputs (batches of long prompts at the large models' feed-forward widths
    come near it): offsets beyond 32 bits into the activations, in rows and in blocks; the first and the last
    rows against float64."""
    m, n, k = 131072 + 256, 256, 16384
    g = torch.Generator(device="cuda:0").manual_seed(3)
    a = torch.empty(m, k, dtype=torch.bfloat16, device="cuda:0")
    for start in range(0, m, 16384):
        a[start:start + 16384] = torch.randn(min(16384, m - start), k, generator=g, device="cuda:0").to(torch.bfloat16)
    w = (torch.randn(n, k, generator=g, device="cuda:0") * 0.02).to(torch.bfloat16)
    packed = K.pack_weight(w)
    assert K.gemm_turns_blocks(m, n, k) == 8
    out = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda:0")
    K.gemm(a, packed, out)                    # regrouped into blocks on the way
    rows = torch.cat([torch.arange(0, 300), torch.arange(m - 300, m)]).to("cuda:0")
    want = a[rows].double() @ w.double().t()
    assert rel(out[rows], want.cpu()) < 4 * math.sqrt(k) * 2.0 ** -24
    assert bool(torch.isfinite(out).all())
    from_rows = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda:0")
    K.gemm_turns(a, packed, from_rows, 8)
    assert torch.equal(out, from_rows)


def test_gemm_with_turns_refuses_what_it_cannot_do(K):
    from beholdd.kernels import KernelError
    a = dev(torch.zeros(256, 192, dtype=torch.bfloat16))
    w = K.pack_weight(dev(torch.zeros(256, 192, dtype=torch.bfloat16)))
    out = torch.empty(256, 256, dtype=torch.float32, device="cuda:0")
    with pytest.raises(KernelError, match="multiple of 128"):
        K.gemm_turns(a, w, out, 8)                                     # K = 192
    a, w = dev(torch.zeros(200, 256, dtype=torch.bfloat16)), K.pack_weight(dev(torch.zeros(256, 256, dtype=torch.bfloat16)))
    with pytest.raises(KernelError, match="M >= 256"):
        K.gemm_turns(a, w, torch.empty(200, 256, dtype=torch.float32, device="cuda:0"), 8)
    a = dev(torch.zeros(256, 256, dtype=torch.bfloat16))
    with pytest.raises(KernelError, match="blocks per wave"):
        K.gemm_turns(a, w, out, 5)
    with pytest.raises(KernelError, match="bfloat16 without accumulation"):
        K.gemm_turns(a, w, torch.empty(256, 256, dtype=torch.bfloat16, device="cuda:0"), 8, accumulate=True)


@pytest.mark.parametrize("m,n,k,swiglu,blocks", [(2048, 6144, 256, False, 6), (2048, 12288, 128, True, 8),
                                                 (2048, 4096, 256, False, 4), (4000, 4096, 128, False, 8),
                                                 (500, 12288, 128, True, 6), (300, 4096, 128, False, 0),
                                                 (512, 151936, 128, False, 8),      # a head over many wanted rows
                                                 (256, 12288, 128, True, 0), (2048, 4096, 12288, False, 0)])
def test_gemm_chooses_the_turns_kernel_where_it_fills_the_chip(K, m, n, k, swiglu, blocks):
    """Which products go to the kernel whose wave groups take turns, and that `gemm` gives the right result there."""
    assert K.gemm_turns_blocks(m, n, k, swiglu) == blocks
    if k > 1024:
        return
    g = torch.Generator().manual_seed(m + n)
    a = torch.randn(m, k, generator=g).to(torch.bfloat16)
    w = (torch.randn(2 * n if swiglu else n, k, generator=g) * 0.05).to(torch.bfloat16)
    packed = K.pack_weight(dev(w))
    if swiglu:
        gate, up = a.double() @ w[:n].double().t(), a.double() @ w[n:].double().t()
        out = torch.empty(m, n, dtype=torch.bfloat16, device="cuda:0")
        K.gemm_swiglu(dev(a), packed, out)
        assert rel(out, gate / (1 + torch.exp(-gate)) * up) < 6e-3
    else:
        want = a.double() @ w.double().t()
        base = torch.randn(m, n, generator=g)
        acc = dev(base.clone())
        K.gemm(dev(a), packed, acc, accumulate=True)
        assert rel(acc, want + base.double()) < 4 * math.sqrt(k) * 2.0 ** -24
        out = torch.empty(m, n, dtype=torch.bfloat16, device="cuda:0")
        K.gemm(dev(a), packed, out)
        assert rel(out, want) < 4e-3


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("m,width,k", [(1, 16, 64), (8, 160, 128), (40, 896, 320), (64, 48, 192), (65, 64, 64),
                                       (130, 208, 256), (300, 1000, 128), (7, 100, 64), (8, 12288, 4096), (5, 32, 72),
                                       (650, 33008, 128), (130, 208, 832), (256, 512, 1024), (100, 256, 512),
                                       (127, 64, 64), (48, 640, 512), (64, 12288, 4096), (33, 136, 1088), (96, 12288, 4096),
                                       (80, 640, 768), (128, 10240, 512)])
def test_gemm_swiglu(K, dtype, packed, m, width, k):
    """silu(a Wg^T) * (a Wu^T) in one pass (or in two where the sizes do not allow one), from both layouts."""
    g = torch.Generator().manual_seed(m + width)
    a = torch.randn(m, k, generator=g).to(dtype)
    w = (torch.randn(2 * width, k, generator=g) * 0.08).to(dtype)
    gate = a.double() @ w[:width].double().t()
    up = a.double() @ w[width:].double().t()
    want = gate / (1 + torch.exp(-gate)) * up
    weight = K.pack_weight(dev(w)) if packed else dev(w)
    out = torch.empty(m, width, dtype=dtype, device="cuda:0")
    K.gemm_swiglu(dev(a), weight, out)
    assert rel(out, want) < tol(dtype, 1e-5, 6e-3), rel(out, want)


def make_cache(n_seqs, lengths, kv_heads, head_dim, dtype, seed, extra_pages=3):
    """Random keys/values for sequences of the given lengths, scattered over shuffled pages.
    Returns (k_pages, v_pages, page_table, dense keys list, dense values list)."""
    g = torch.Generator().manual_seed(seed)
    pages_per = [-(-n // PAGE) for n in lengths]
    n_pages = sum(pages_per) + extra_pages
    order = torch.randperm(n_pages, generator=g).tolist()
    k_pages = torch.randn(n_pages, kv_heads, PAGE, head_dim, generator=g).to(dtype)   # garbage everywhere
    v_pages = torch.randn(n_pages, kv_heads, head_dim, PAGE, generator=g).to(dtype)           # transposed in a page
    width = max(pages_per)
    table = torch.zeros(n_seqs, width, dtype=torch.int32)
    keys, values = [], []
    for s, n in enumerate(lengths):
        mine = [order.pop() for _ in range(pages_per[s])]
        table[s, :len(mine)] = torch.tensor(mine, dtype=torch.int32)
        k = torch.randn(n, kv_heads, head_dim, generator=g).to(dtype)
        v = torch.randn(n, kv_heads, head_dim, generator=g).to(dtype)
        for p in range(n):
            k_pages[mine[p // PAGE], :, p % PAGE] = k[p]
            v_pages[mine[p // PAGE], :, :, p % PAGE] = v[p]
        keys.append(k)
        values.append(v)
    return k_pages, v_pages, table, keys, values


def piece_order(head_dim):
    """Where key [token, dim] and value [dim, token] lie within one head's share of a page when the cache
    is kept in 16-byte pieces: written from the description of that order, piece by piece, not from the
    kernels' index arithmetic.  Piece (t * head_dim/32 + s) * 64 + lane of the keys holds token
    32 (t/2) + 4 (t%2) + 8 (j/4) + j%4, dims 32 s + 8 g .. + 7 (lane = 16 g + j); piece (dt * 2 + u) * 64 +
    lane of the values holds dim 16 dt + j, tokens 32 u + 8 g .. + 7."""
    k_at = torch.full((PAGE, head_dim), -1, dtype=torch.long)
    v_at = torch.full((head_dim, PAGE), -1, dtype=torch.long)
    slices = head_dim // 32
    for lane in range(64):
        g, j = lane // 16, lane % 16
        for t in range(4):
            token = 32 * (t // 2) + 4 * (t % 2) + 8 * (j // 4) + j % 4
            for s in range(slices):
                piece = (t * slices + s) * 64 + lane
                for e in range(8):
                    k_at[token, 32 * s + 8 * g + e] = piece * 8 + e
        for dt in range(head_dim // 16):
            for u in range(2):
                piece = (dt * 2 + u) * 64 + lane
                for e in range(8):
                    v_at[16 * dt + j, 32 * u + 8 * g + e] = piece * 8 + e
    assert sorted(k_at.reshape(-1).tolist()) == list(range(PAGE * head_dim))       # a permutation
    assert sorted(v_at.reshape(-1).tolist()) == list(range(PAGE * head_dim))
    return k_at.reshape(-1), v_at.reshape(-1)


def stored(K, k_pages, v_pages):
    """Pages given as keys [.., token, dim] and values [.., dim, token], on the device in the order the
    kernels keep them for this element type and head size."""
    head_dim = k_pages.shape[-1]
    if K.kv_order(k_pages.dtype, head_dim) == 0:
        return dev(k_pages), dev(v_pages)
    k_at, v_at = piece_order(head_dim)
    lead = k_pages.shape[:2]
    ks, vs = torch.empty_like(k_pages).reshape(*lead, -1), torch.empty_like(v_pages).reshape(*lead, -1)
    ks[..., k_at] = k_pages.cpu().reshape(*lead, -1)
    vs[..., v_at] = v_pages.cpu().reshape(*lead, -1)
    return dev(ks.reshape(k_pages.shape)), dev(vs.reshape(v_pages.shape))


def as_rows(K, k_stored, v_stored):
    """The inverse of `stored`, on the CPU."""
    head_dim = k_stored.shape[-1]
    k_stored, v_stored = k_stored.cpu(), v_stored.cpu()
    if K.kv_order(k_stored.dtype, head_dim) == 0:
        return k_stored, v_stored
    k_at, v_at = piece_order(head_dim)
    lead = k_stored.shape[:2]
    return (k_stored.reshape(*lead, -1)[..., k_at].reshape(k_stored.shape),
            v_stored.reshape(*lead, -1)[..., v_at].reshape(v_stored.shape))


def attention_reference(q, keys, values, pos, n_heads, kv_heads, head_dim, scale, window):
    group = n_heads // kv_heads
    first = max(0, pos - window + 1) if window else 0
    out = torch.empty(n_heads, head_dim, dtype=torch.float64)
    for h in range(n_heads):
        k = keys[first:pos + 1, h // group].double()
        v = values[first:pos + 1, h // group].double()
        p = torch.softmax(k @ q[h].double() * scale, 0)
        out[h] = p @ v
    return out


class Layout:
    def __init__(self, is_decode, seq_start, n_seqs, max_rows_per_seq, max_position):
        self.is_decode, self.seq_start, self.n_seqs = is_decode, seq_start, n_seqs
        self.max_rows_per_seq, self.max_position = max_rows_per_seq, max_position


ATTN_SHAPES = [  # heads, kv heads, head size
    (4, 2, 16), (6, 2, 48), (8, 8, 64), (5, 1, 80), (8, 2, 128), (3, 3, 256), (12, 4, 96), (14, 2, 128),
    (32, 1, 64), (40, 2, 32),          # 32 and 20 query heads to a kv head: more than one tile of columns shares a head
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n_heads,kv_heads,head_dim", ATTN_SHAPES)
@pytest.mark.parametrize("window", [0, 70])
def test_attention_decode_rows(K, dtype, n_heads, kv_heads, head_dim, window):
    """One query per sequence at the end of caches of unequal lengths (page edges included)."""
    lengths = [1, 63, 64, 65, 130, 517]
    kp, vp, table, keys, values = make_cache(len(lengths), lengths, kv_heads, head_dim, dtype, seed=head_dim + n_heads)
    g = torch.Generator().manual_seed(7)
    q = torch.randn(len(lengths), n_heads * head_dim, generator=g).to(dtype)
    positions = torch.tensor([n - 1 for n in lengths], dtype=torch.int32)
    row_seq = torch.arange(len(lengths), dtype=torch.int32)
    out = torch.empty(len(lengths), n_heads * head_dim, dtype=dtype, device="cuda:0")
    scale = 1 / math.sqrt(head_dim)
    layout = Layout(True, dev(torch.arange(len(lengths) + 1, dtype=torch.int32)), len(lengths), 1, max(lengths) - 1)
    K.attention(dev(q), out, *stored(K, kp, vp), dev(table), dev(row_seq), dev(positions), n_heads, kv_heads,
                head_dim, scale, window, layout=layout)
    for s, n in enumerate(lengths):
        want = attention_reference(q[s].reshape(n_heads, head_dim), keys[s], values[s], n - 1, n_heads, kv_heads,
                                   head_dim, scale, window)
        assert rel(out[s].reshape(n_heads, head_dim), want) < tol(dtype, 1e-5, 1.2e-2), (s, n)


@pytest.mark.parametrize("n_heads,kv_heads,head_dim", [(8, 2, 128), (4, 4, 64), (6, 1, 96), (32, 8, 128)])
def test_attention_decode_with_split_keys_and_garbage_beyond_the_end(K, n_heads, kv_heads, head_dim):
    """Long caches and few sequences: the keys are split over workgroups and combined.  Whatever lies in
    a page beyond a sequence's last token (here NaN) must not reach the result."""
    dtype = torch.bfloat16
    lengths = [3000, 1, 1500, 2049]
    kp, vp, table, keys, values = make_cache(len(lengths), lengths, kv_heads, head_dim, dtype, seed=head_dim)
    for s, n in enumerate(lengths):
        if n % PAGE:
            page = int(table[s, (n - 1) // PAGE])
            kp[page, :, n % PAGE:, :] = float("nan")
            vp[page, :, :, n % PAGE:] = float("nan")
    g = torch.Generator().manual_seed(3)
    q = torch.randn(len(lengths), n_heads * head_dim, generator=g).to(dtype)
    positions = torch.tensor([n - 1 for n in lengths], dtype=torch.int32)
    row_seq = torch.arange(len(lengths), dtype=torch.int32)
    out = torch.empty(len(lengths), n_heads * head_dim, dtype=dtype, device="cuda:0")
    scale = 1 / math.sqrt(head_dim)
    layout = Layout(True, dev(torch.arange(len(lengths) + 1, dtype=torch.int32)), len(lengths), 1, max(lengths) - 1)
    assert K.lib.bh_attention_bf16_splits(len(lengths), 1, n_heads, kv_heads, max(lengths) - 1) > 1
    K.attention(dev(q), out, *stored(K, kp, vp), dev(table), dev(row_seq), dev(positions), n_heads, kv_heads,
                head_dim, scale, 0, layout=layout)
    assert bool(torch.isfinite(out.float()).all())
    for s, n in enumerate(lengths):
        want = attention_reference(q[s].reshape(n_heads, head_dim), keys[s], values[s], n - 1, n_heads, kv_heads,
                                   head_dim, scale, 0)
        assert rel(out[s].reshape(n_heads, head_dim), want) < 1.2e-2, (s, n)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n_heads,kv_heads,head_dim", ATTN_SHAPES)
def test_attention_prefill_rows_ragged(K, dtype, n_heads, kv_heads, head_dim):
    """Several sequences in one step: new tokens after pasts of different lengths (0 included)."""
    pasts, news = [0, 5, 64, 100, 0], [70, 1, 3, 131, 1]
    lengths = [p + n for p, n in zip(pasts, news)]
    kp, vp, table, keys, values = make_cache(len(lengths), lengths, kv_heads, head_dim, dtype, seed=3 * head_dim + n_heads)
    g = torch.Generator().manual_seed(11)
    n_rows = sum(news)
    q = torch.randn(n_rows, n_heads * head_dim, generator=g).to(dtype)
    positions = torch.tensor([p + t for p, n in zip(pasts, news) for t in range(n)], dtype=torch.int32)
    row_seq = torch.tensor([s for s, n in enumerate(news) for _ in range(n)], dtype=torch.int32)
    starts = torch.tensor(np.concatenate([[0], np.cumsum(news)]), dtype=torch.int32)
    out = torch.empty(n_rows, n_heads * head_dim, dtype=dtype, device="cuda:0")
    scale = 1 / math.sqrt(head_dim)
    K.attention(dev(q), out, *stored(K, kp, vp), dev(table), dev(row_seq), dev(positions), n_heads, kv_heads,
                head_dim, scale, 0, layout=Layout(False, dev(starts), len(lengths), max(news), max(lengths) - 1))
    worst = 0.0
    for row in range(n_rows):
        s = int(row_seq[row])
        want = attention_reference(q[row].reshape(n_heads, head_dim), keys[s], values[s], int(positions[row]),
                                   n_heads, kv_heads, head_dim, scale, 0)
        worst = max(worst, rel(out[row].reshape(n_heads, head_dim), want))
    assert worst < tol(dtype, 1e-5, 1.2e-2), worst


def attention_reference_rows(q, keys, values, positions, n_heads, kv_heads, head_dim, scale, window):
    """All rows of one sequence at once: q [rows, heads * head_dim], row r at position positions[r]."""
    rows, group = q.shape[0], n_heads // kv_heads
    qh = q.double().reshape(rows, kv_heads, group, head_dim)
    scores = torch.einsum("rkgd,nkd->rkgn", qh, keys.double()) * scale
    key_at = torch.arange(keys.shape[0])[None, :]
    hidden = key_at > positions[:, None]
    if window:
        hidden |= key_at < positions[:, None] - window + 1
    scores = scores.masked_fill(hidden[:, None, None, :], float("-inf"))
    return torch.einsum("rkgn,nkd->rkgd", torch.softmax(scores, -1), values.double()).reshape(rows, n_heads * head_dim)


@pytest.mark.parametrize("window", [0, 100])
@pytest.mark.parametrize("n_heads,kv_heads,head_dim", [(32, 8, 128), (8, 2, 64), (6, 1, 96), (4, 4, 256), (2, 2, 32),
                                                       (4, 2, 160)])
@pytest.mark.parametrize("copies", [1, 5])
def test_attention_prefill_many_columns(K, n_heads, kv_heads, head_dim, window, copies):
    """Steps wide enough for the kernel that keeps a page in LDS for four waves with columns of their own:
    several sequences with pasts, ends that fill neither a tile nor a workgroup, NaN beyond the last key.
    Five copies of the sequences make enough workgroups for two column tiles per wave, one copy runs with one."""
    dtype = torch.bfloat16
    group = n_heads // kv_heads
    longest = -(-1024 * 16 // (n_heads * 3)) + 40
    pasts, news = [0, 70, 129] * copies, [longest, longest // 2 + 3, 65] * copies
    assert -(-max(news) * group // 16) * kv_heads * 3 >= 1024      # what sends a step to that kernel
    assert (-(-max(news) * group // 128) * kv_heads * len(news) >= 512) == (copies == 5)
    lengths = [p + n for p, n in zip(pasts, news)]
    kp, vp, table, keys, values = make_cache(len(lengths), lengths, kv_heads, head_dim, dtype, seed=head_dim + n_heads)
    for s, n in enumerate(lengths):
        if n % PAGE:
            page = int(table[s, (n - 1) // PAGE])
            kp[page, :, n % PAGE:, :] = float("nan")
            vp[page, :, :, n % PAGE:] = float("nan")
    g = torch.Generator().manual_seed(13)
    n_rows = sum(news)
    q = torch.randn(n_rows, n_heads * head_dim, generator=g).to(dtype)
    positions = torch.tensor([p + t for p, n in zip(pasts, news) for t in range(n)], dtype=torch.int32)
    row_seq = torch.tensor([s for s, n in enumerate(news) for _ in range(n)], dtype=torch.int32)
    starts = torch.tensor(np.concatenate([[0], np.cumsum(news)]), dtype=torch.int32)
    out = torch.empty(n_rows, n_heads * head_dim, dtype=dtype, device="cuda:0")
    scale = 1 / math.sqrt(head_dim)
    K.attention(dev(q), out, *stored(K, kp, vp), dev(table), dev(row_seq), dev(positions), n_heads, kv_heads,
                head_dim, scale, window, layout=Layout(False, dev(starts), len(lengths), max(news), max(lengths) - 1))
    assert bool(torch.isfinite(out.float()).all())
    for s in range(len(news)):
        rows = slice(int(starts[s]), int(starts[s + 1]))
        want = attention_reference_rows(q[rows], keys[s], values[s], positions[rows].long(), n_heads, kv_heads,
                                        head_dim, scale, window)
        assert rel(out[rows], want) < 1.2e-2, (s, rel(out[rows], want))
    from beholdd.kernels.library import BlockedRows     # the same output in blocks of 16 rows x 32 columns
    width = n_heads * head_dim
    blocked = BlockedRows(torch.full((-(-n_rows // 256) * 256 * width,), float("nan"), dtype=dtype, device="cuda:0"), n_rows, width)
    K.attention(dev(q), blocked, *stored(K, kp, vp), dev(table), dev(row_seq), dev(positions), n_heads, kv_heads,
                head_dim, scale, window, layout=Layout(False, dev(starts), len(lengths), max(news), max(lengths) - 1))
    assert torch.equal(K.from_blocked(blocked), out)


@pytest.mark.parametrize("n_heads,kv_heads,head_dim", [(32, 8, 128), (16, 4, 64)])
def test_attention_prefill_when_the_largest_score_keeps_growing(K, n_heads, kv_heads, head_dim):
    """One direction is planted in every query and in the keys with a weight that grows along the sequence: by a
    little from key to key (the largest score so far grows by less than a factor of two a page), then twentyfold
    from one key on (a jump by more than two hundred powers of two, which no float32 holds).  The kernel that keeps
    the exponentials' reference while the maximum grows little has to follow both: a reference not moved at the jump
    gives infinite probabilities, one moved without scaling what was summed before gives wrong rows after it."""
    dtype = torch.bfloat16
    n = 1500
    g = torch.Generator().manual_seed(head_dim)
    kp, vp, table, keys, values = make_cache(1, [n], kv_heads, head_dim, dtype, seed=7)
    direction = torch.randn(head_dim, generator=g)
    direction /= direction.norm()
    weight = 0.02 * torch.arange(n, dtype=torch.float32)             # scores along the direction grow by 0.02 * |q.d| * scale a key
    weight[1100:] *= 20.0
    planted = (keys[0].float() * 0.3 + weight[:, None, None] * direction).to(dtype)
    keys[0] = planted
    for t in range(n):
        kp[int(table[0, t // PAGE]), :, t % PAGE] = planted[t]
    q = (torch.randn(n, n_heads, head_dim, generator=g) * 0.3 + 4.0 * direction).to(dtype).reshape(n, n_heads * head_dim)
    positions = torch.arange(n, dtype=torch.int32)
    starts = torch.tensor([0, n], dtype=torch.int32)
    scale = 1 / math.sqrt(head_dim)
    assert -(-n * (n_heads // kv_heads) // 16) * kv_heads >= 1024      # what sends the step to the kernel for many columns
    out = torch.empty(n, n_heads * head_dim, dtype=dtype, device="cuda:0")
    K.attention(dev(q), out, *stored(K, kp, vp), dev(table), dev(torch.zeros(n, dtype=torch.int32)), dev(positions),
                n_heads, kv_heads, head_dim, scale, 0, layout=Layout(False, dev(starts), 1, n, n - 1))
    want = attention_reference_rows(q, keys[0], values[0], positions.long(), n_heads, kv_heads, head_dim, scale, 0)
    for rows in (slice(0, 64), slice(64, 1100), slice(1100, 1164), slice(1164, n)):
        assert rel(out[rows], want[rows]) < 1.2e-2, (rows, rel(out[rows], want[rows]))


@pytest.mark.parametrize("window", [0, 70])
@pytest.mark.parametrize("with_norm,with_rope,write_kv", [(True, True, True), (False, True, True), (True, False, True),
                                                          (True, True, False)])
@pytest.mark.parametrize("n_heads,kv_heads,head_dim", [(32, 8, 128), (8, 2, 64), (4, 4, 128), (6, 1, 256), (16, 1, 64)])
def test_decode_attention_from_the_projection_rows(K, n_heads, kv_heads, head_dim, with_norm, with_rope, write_kv, window):
    """Norm, rotation, cache write and attention of a decode step in one launch give what the two launches
    give: the same output and the same cache, for sequences at a page's first and last slot, at position 0,
    and long enough for split keys."""
    dtype = torch.bfloat16
    lengths = [1, 64, 65, 128, 131, 2500, 700]             # the new token stands at length - 1
    n = len(lengths)
    kp, vp, table, keys, values = make_cache(n, lengths, kv_heads, head_dim, dtype, seed=head_dim + n_heads)
    gen = torch.Generator().manual_seed(5)
    qkv = torch.randn(n, (n_heads + 2 * kv_heads) * head_dim, generator=gen).to(dtype)
    qw = kw = cos = sin = None
    if with_norm:
        qw = dev((1 + 0.2 * torch.randn(head_dim, generator=gen)).to(dtype))
        kw = dev((1 + 0.2 * torch.randn(head_dim, generator=gen)).to(dtype))
    if with_rope:
        freqs = 1.0 / 10000.0 ** (torch.arange(0, head_dim, 2, dtype=torch.float64) / head_dim)
        angles = torch.arange(2600, dtype=torch.float64)[:, None] * freqs
        cos, sin = dev(angles.cos().float()), dev(angles.sin().float())
    positions = dev(torch.tensor([length - 1 for length in lengths], dtype=torch.int32))
    row_seq = dev(torch.arange(n, dtype=torch.int32))
    layout = Layout(True, dev(torch.arange(n + 1, dtype=torch.int32)), n, 1, max(lengths) - 1)
    scale, eps = 1 / math.sqrt(head_dim), 1e-5

    k_two, v_two = stored(K, kp, vp)
    q = torch.empty(n, n_heads * head_dim, dtype=dtype, device="cuda:0")
    out_two = torch.empty_like(q)
    K.qk_norm_rope_cache(dev(qkv), q, qw, kw, eps, cos, sin, positions, row_seq, k_two, v_two, dev(table), n_heads,
                         kv_heads, head_dim, write_kv, max(lengths) - 1)
    K.attention(q, out_two, k_two, v_two, dev(table), row_seq, positions, n_heads, kv_heads, head_dim, scale, window,
                layout=layout)

    k_one, v_one = stored(K, kp, vp)
    out_one = torch.empty_like(q)
    took = K.attention_decode_fused(dev(qkv), out_one, qw, kw, eps, cos, sin, positions, k_one, v_one, dev(table),
                                    n_heads, kv_heads, head_dim, scale, window, write_kv, layout)
    assert took is True
    assert bool(torch.isfinite(out_one.float()).all())
    assert rel(out_one, out_two.double()) < 8e-3, rel(out_one, out_two.double())
    assert torch.equal(v_one.cpu(), v_two.cpu())
    assert rel(k_one, k_two.double()) < 8e-3                  # the same numbers but for the order of two float32 sums
    assert (k_one.cpu() != k_two.cpu()).float().mean() < 1e-3
    if not write_kv:
        assert torch.equal(k_one.cpu(), stored(K, kp, vp)[0].cpu())
    from beholdd.kernels.library import BlockedRows      # the same output in blocks of 8 and of 16 rows
    width = n_heads * head_dim
    for block_rows in (8, 16):
        k_b, v_b = stored(K, kp, vp)
        blocked = BlockedRows(torch.full((16 * width,), float("nan"), dtype=dtype, device="cuda:0"), n, width, block_rows)
        assert K.attention_decode_fused(dev(qkv), blocked, qw, kw, eps, cos, sin, positions, k_b, v_b, dev(table),
                                        n_heads, kv_heads, head_dim, scale, window, write_kv, layout) is True
        assert torch.equal(K.from_blocked(blocked), out_one)
        # and from finished queries, by the kernels for few columns (a step of seven rows here)
        K.attention(q, blocked, k_two, v_two, dev(table), row_seq, positions, n_heads, kv_heads, head_dim, scale, window,
                    layout=layout)
        assert torch.equal(K.from_blocked(blocked), out_two)


def test_decode_attention_from_the_projection_rows_of_many_sequences(K):
    """Forty sequences on eight kv heads: more workgroups than compute units, no split keys; the one launch runs in
    the form that norms the queries before the first page and takes the new key's numbers after the last."""
    dtype, n_heads, kv_heads, head_dim = torch.bfloat16, 32, 8, 128
    lengths = [1 + (37 * i) % 300 for i in range(40)]
    n = len(lengths)
    kp, vp, table, keys, values = make_cache(n, lengths, kv_heads, head_dim, dtype, seed=9)
    gen = torch.Generator().manual_seed(6)
    qkv = torch.randn(n, (n_heads + 2 * kv_heads) * head_dim, generator=gen).to(dtype)
    qw = dev((1 + 0.2 * torch.randn(head_dim, generator=gen)).to(dtype))
    kw = dev((1 + 0.2 * torch.randn(head_dim, generator=gen)).to(dtype))
    freqs = 1.0 / 1e6 ** (torch.arange(0, head_dim, 2, dtype=torch.float64) / head_dim)
    angles = torch.arange(512, dtype=torch.float64)[:, None] * freqs
    cos, sin = dev(angles.cos().float()), dev(angles.sin().float())
    positions = dev(torch.tensor([length - 1 for length in lengths], dtype=torch.int32))
    row_seq = dev(torch.arange(n, dtype=torch.int32))
    layout = Layout(True, dev(torch.arange(n + 1, dtype=torch.int32)), n, 1, max(lengths) - 1)
    assert K.lib.bh_attention_bf16_splits(n, 1, n_heads, kv_heads, max(lengths) - 1) == 1
    scale, eps = 1 / math.sqrt(head_dim), 1e-6
    k_two, v_two = stored(K, kp, vp)
    q = torch.empty(n, n_heads * head_dim, dtype=dtype, device="cuda:0")
    out_two = torch.empty_like(q)
    K.qk_norm_rope_cache(dev(qkv), q, qw, kw, eps, cos, sin, positions, row_seq, k_two, v_two, dev(table), n_heads,
                         kv_heads, head_dim, True, max(lengths) - 1)
    K.attention(q, out_two, k_two, v_two, dev(table), row_seq, positions, n_heads, kv_heads, head_dim, scale, 0, layout=layout)
    k_one, v_one = stored(K, kp, vp)
    out_one = torch.empty_like(q)
    assert K.attention_decode_fused(dev(qkv), out_one, qw, kw, eps, cos, sin, positions, k_one, v_one, dev(table), n_heads,
                                    kv_heads, head_dim, scale, 0, True, layout) is True
    assert rel(out_one, out_two.double()) < 8e-3
    assert torch.equal(v_one.cpu(), v_two.cpu()) and rel(k_one, k_two.double()) < 8e-3
    # and against the plain attention over the dense keys and values, with the new key and value in place
    k_rows, v_rows = as_rows(K, k_one, v_one)
    for s in (0, 7, 39):
        pos = lengths[s] - 1
        page = int(table[s, pos // PAGE])
        keys[s][pos] = k_rows[page, :, pos % PAGE].float().to(dtype)
        values[s][pos] = v_rows[page, :, :, pos % PAGE].float().to(dtype)
        want = attention_reference(q[s].cpu().reshape(n_heads, head_dim), keys[s], values[s], pos, n_heads, kv_heads, head_dim, scale, 0)
        assert rel(out_one[s].reshape(n_heads, head_dim), want) < 1.2e-2, s


def test_decode_attention_from_the_projection_rows_says_when_it_cannot(K):
    dtype = torch.bfloat16
    kp, vp, table, _, _ = make_cache(1, [10], 2, 48, dtype, seed=1)
    qkv = dev(torch.randn(1, 8 * 48).to(dtype))
    out = torch.empty(1, 4 * 48, dtype=dtype, device="cuda:0")
    layout = Layout(True, dev(torch.tensor([0, 1], dtype=torch.int32)), 1, 1, 9)
    positions = dev(torch.tensor([9], dtype=torch.int32))
    k_pages, v_pages = stored(K, kp, vp)
    assert K.attention_decode_fused(qkv, out, None, None, 0.0, None, None, positions, k_pages, v_pages, dev(table),
                                    4, 2, 48, 0.1, 0, True, layout) is False          # head size 48


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("far", [0, 63, 64, 127, 128, 300, 511, 640])
def test_attention_finds_one_far_key_among_hundreds(K, dtype, far):
    """The query and one key are made to fit each other so that this key takes all the weight:
    the output must be that key's value, wherever in the pages it lies."""
    n_heads, kv_heads, head_dim, n = 4, 2, 64, 700
    kp, vp, table, keys, values = make_cache(1, [n], kv_heads, head_dim, dtype, seed=far)
    q = torch.zeros(2, n_heads, head_dim)
    direction = torch.nn.functional.normalize(torch.randn(head_dim, generator=torch.Generator().manual_seed(1)), dim=0)
    q[:] = direction * 30
    page = int(table[0, far // PAGE])
    kp[page, :, far % PAGE] = (direction * 30).to(dtype)
    keys[0][far] = (direction * 30).to(dtype)
    q = q.reshape(2, n_heads * head_dim).to(dtype)
    positions = torch.tensor([n - 1, max(far, 1)], dtype=torch.int32)      # the last row sees the key as its newest
    row_seq = torch.zeros(2, dtype=torch.int32)
    grouped = Layout(False, dev(torch.tensor([0, 2], dtype=torch.int32)), 1, 2, n - 1)
    for layout in (None, grouped):          # the kernel for any size, and the matrix-core kernel
        out = torch.empty(2, n_heads * head_dim, dtype=dtype, device="cuda:0")
        K.attention(dev(q), out, *stored(K, kp, vp), dev(table), dev(row_seq), dev(positions), n_heads, kv_heads,
                    head_dim, 1 / math.sqrt(head_dim), 0, layout=layout)
        got = out.float().cpu().reshape(2, n_heads, head_dim)
        for h in range(n_heads):
            assert torch.allclose(got[0, h], values[0][far, h // 2].float(), atol=2e-2), (far, h, layout)
            assert torch.allclose(got[1, h], values[0][far, h // 2].float(), atol=2e-2), (far, h, layout)


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_window_edge(K, dtype):
    """A key just outside the window must be invisible, the one just inside visible."""
    n_heads, kv_heads, head_dim, n, window = 2, 1, 32, 200, 70
    kp, vp, table, keys, values = make_cache(1, [n], kv_heads, head_dim, dtype, seed=5)
    direction = torch.ones(head_dim) / math.sqrt(head_dim)
    pos = n - 1
    outside, inside = pos - window, pos - window + 1
    for where in (outside, inside):
        page = int(table[0, where // PAGE])
        kp[page, :, where % PAGE] = (direction * (40 if where == outside else 25)).to(dtype)
    q = (direction * 30).repeat(n_heads).reshape(1, -1).to(dtype)
    out = torch.empty(1, n_heads * head_dim, dtype=dtype, device="cuda:0")
    args = (*stored(K, kp, vp), dev(table), dev(torch.zeros(1, dtype=torch.int32)), dev(torch.tensor([pos], dtype=torch.int32)),
            n_heads, kv_heads, head_dim, 1 / math.sqrt(head_dim))
    K.attention(dev(q), out, *args, window)
    assert torch.allclose(out.float().cpu().reshape(n_heads, head_dim)[0], values[0][inside, 0].float(), atol=2e-2)
    K.attention(dev(q), out, *args, 0)
    assert torch.allclose(out.float().cpu().reshape(n_heads, head_dim)[0], values[0][outside, 0].float(), atol=2e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("w_dtype", DTYPES)
# few rows; enough for the kernel for many rows; and the same with a sequence whose whole pieces of eight tokens
# begin at rows 3, 11, ... and steps that begin and end inside a piece
@pytest.mark.parametrize("news,pasts", [([3, 5, 1], [0, 62, 130]), ([70, 5, 1], [0, 62, 130]), ([3, 70, 2], [5, 16, 7])])
@pytest.mark.parametrize("n_heads,kv_heads,head_dim,rot", [(4, 2, 16, 16), (6, 2, 48, 48), (5, 1, 80, 32),
                                                           (8, 2, 128, 128), (3, 3, 256, 256), (5, 1, 64, 64),
                                                           (5, 1, 128, 0), (7, 7, 128, 128), (4, 2, 128, 64)])
def test_qk_norm_rope_cache(K, dtype, w_dtype, n_heads, kv_heads, head_dim, rot, news, pasts):
    g = torch.Generator().manual_seed(head_dim)
    n_rows = sum(news)
    fused = (n_heads + 2 * kv_heads) * head_dim
    qkv = torch.randn(n_rows, fused, generator=g).to(dtype)
    qw = (1 + 0.2 * torch.randn(head_dim, generator=g)).to(w_dtype)
    kw = (1 + 0.2 * torch.randn(head_dim, generator=g)).to(w_dtype)
    eps, theta, max_pos = 1e-5, 10000.0, 256
    freqs = 1.0 / theta ** (torch.arange(0, rot, 2, dtype=torch.float64) / rot)
    angles = torch.arange(max_pos, dtype=torch.float64)[:, None] * freqs
    cos, sin = angles.cos().float(), angles.sin().float()
    positions = torch.tensor([p + t for p, n in zip(pasts, news) for t in range(n)], dtype=torch.int32)
    row_seq = torch.tensor([s for s, n in enumerate(news) for _ in range(n)], dtype=torch.int32)
    n_pages = 9
    table = torch.tensor([[4, 5, 0], [7, 2, 0], [1, 8, 3]], dtype=torch.int32)
    sentinel = 768.0        # exact in bfloat16
    kp = torch.full((n_pages, kv_heads, PAGE, head_dim), sentinel).to(dtype)
    vp = torch.full((n_pages, kv_heads, head_dim, PAGE), sentinel).to(dtype)
    kp_d, vp_d = stored(K, kp, vp)
    q_out = torch.empty(n_rows, n_heads * head_dim, dtype=dtype, device="cuda:0")
    K.qk_norm_rope_cache(dev(qkv), q_out, dev(qw), dev(kw), eps, dev(cos), dev(sin), dev(positions), dev(row_seq),
                         kp_d, vp_d, dev(table), n_heads, kv_heads, head_dim, True, int(positions.max()))

    def reference(x, w, pos):      # x [heads, head_dim] float64
        y = x / torch.sqrt((x ** 2).mean(-1, keepdim=True) + eps) * w.double()
        half = rot // 2
        c, s = cos[pos].double(), sin[pos].double()
        a, b = y[:, :half], y[:, half:rot]
        return torch.cat([a * c - b * s, a * s + b * c, y[:, rot:]], dim=-1)

    written = torch.zeros(n_pages, PAGE, dtype=torch.bool)
    kp_d, vp_d = as_rows(K, kp_d, vp_d)
    for row in range(n_rows):
        pos, seq = int(positions[row]), int(row_seq[row])
        x = qkv[row].double()
        q_want = reference(x[:n_heads * head_dim].reshape(n_heads, head_dim), qw, pos)
        k_want = reference(x[n_heads * head_dim:(n_heads + kv_heads) * head_dim].reshape(kv_heads, head_dim), kw, pos)
        v_want = x[(n_heads + kv_heads) * head_dim:].reshape(kv_heads, head_dim)
        page = int(table[seq, pos // PAGE])
        written[page, pos % PAGE] = True
        assert rel(q_out[row].reshape(n_heads, head_dim), q_want) < tol(dtype, 2e-6, 4e-3)
        assert rel(kp_d[page, :, pos % PAGE], k_want) < tol(dtype, 2e-6, 4e-3)
        assert torch.equal(vp_d[page, :, :, pos % PAGE].cpu().double(), v_want)
    # nothing else in the cache was touched
    untouched = ~written[:, None, :, None].expand(n_pages, kv_heads, PAGE, head_dim)
    assert bool((kp_d.cpu().float()[untouched] == sentinel).all())
    assert bool((vp_d.cpu().float().transpose(2, 3)[untouched] == sentinel).all())
    # without weights and tables the heads pass through; without write_kv the cache stays as it is
    kp2, vp2 = stored(K, kp, vp)
    K.qk_norm_rope_cache(dev(qkv), q_out, None, None, 0.0, None, None, dev(positions), dev(row_seq), kp2, vp2,
                         dev(table), n_heads, kv_heads, head_dim, False, int(positions.max()))
    assert torch.equal(q_out.cpu(), qkv[:, :n_heads * head_dim])
    assert torch.equal(kp2.cpu(), kp) and torch.equal(vp2.cpu(), vp)


def test_qk_norm_rope_cache_takes_rows_in_any_order(K):
    """The kernel for many rows writes whole pieces of eight values only where the eight positions are consecutive rows;
    rows of two sequences interleaved, a sequence's rows backwards and a gap in the positions land where they belong."""
    n_heads, kv_heads, head_dim = 8, 2, 128
    g = torch.Generator().manual_seed(5)
    # sequence 0: positions 0..39 interleaved with sequence 1's 64..103 backwards; sequence 2: 8..23 then 32..39
    order = []
    for t in range(40):
        order += [(0, t), (1, 103 - t)]
    order += [(2, p) for p in list(range(8, 24)) + list(range(32, 40))]
    n_rows = len(order)
    row_seq = torch.tensor([s for s, _ in order], dtype=torch.int32)
    positions = torch.tensor([p for _, p in order], dtype=torch.int32)
    fused = (n_heads + 2 * kv_heads) * head_dim
    qkv = torch.randn(n_rows, fused, generator=g).to(torch.bfloat16)
    table = torch.tensor([[4, 5], [7, 2], [1, 8]], dtype=torch.int32)
    results = []
    for permuted in (False, True):      # the same rows sorted by (sequence, position): the kernel's pieces of eight
        index = sorted(range(n_rows), key=lambda r: order[r]) if permuted else list(range(n_rows))
        kp = torch.full((9, kv_heads, PAGE, head_dim), 768.0).to(torch.bfloat16)
        vp = torch.full((9, kv_heads, head_dim, PAGE), 768.0).to(torch.bfloat16)
        kp_d, vp_d = stored(K, kp, vp)
        q_out = torch.empty(n_rows, n_heads * head_dim, dtype=torch.bfloat16, device="cuda:0")
        K.qk_norm_rope_cache(dev(qkv[index]), q_out, None, None, 0.0, None, None, dev(positions[index]), dev(row_seq[index]),
                             kp_d, vp_d, dev(table), n_heads, kv_heads, head_dim, True, 103)
        back = torch.empty_like(q_out)
        back[torch.tensor(index, device="cuda:0")] = q_out
        kp_r, vp_r = as_rows(K, kp_d, vp_d)
        results.append((back.cpu(), kp_r.cpu(), vp_r.cpu()))
    for any_order, sorted_rows in zip(*results):
        assert torch.equal(any_order, sorted_rows)
    kp_r, vp_r = results[0][1], results[0][2]
    for row, (seq, pos) in enumerate(order):
        page = int(table[seq, pos // PAGE])
        want_v = qkv[row, (n_heads + kv_heads) * head_dim:].reshape(kv_heads, head_dim)
        assert torch.equal(vp_r[page, :, :, pos % PAGE], want_v)
        assert torch.equal(kp_r[page, :, pos % PAGE], qkv[row, n_heads * head_dim:(n_heads + kv_heads) * head_dim].reshape(kv_heads, head_dim))


@pytest.mark.parametrize("w_dtype", DTYPES)
@pytest.mark.parametrize("parts", [2, 4, 8])
@pytest.mark.parametrize("news,pasts", [([70, 5, 1], [0, 62, 130]), ([3, 70, 2], [5, 16, 7]), ([66, 5, 6], [0, 62, 130])])
@pytest.mark.parametrize("n_heads,kv_heads,head_dim,rot", [(8, 2, 128, 128), (3, 3, 256, 256), (5, 1, 64, 64), (5, 1, 128, 0)])
def test_qk_norm_rope_cache_from_the_sums_of_a_products_parts(K, w_dtype, parts, news, pasts, n_heads, kv_heads, head_dim, rot):
    """The same kernel fed with the float32 sums of K's parts instead of finished bfloat16 rows writes, bit for bit,
    what it writes from the rows that the parts add up to (in their order, rounded to bfloat16)."""
    from beholdd.kernels import PartSums
    g = torch.Generator().manual_seed(head_dim + parts)
    n_rows = sum(news)
    fused = (n_heads + 2 * kv_heads) * head_dim
    sums = torch.randn(parts, n_rows, fused, generator=g) * torch.tensor([1.0, -0.7, 0.3, 2.0, 0.1, -1.3, 0.6, 0.9][:parts])[:, None, None]
    total = torch.zeros(n_rows, fused)
    for part in range(parts):
        total = total + sums[part]
    rows = total.to(torch.bfloat16)
    qw = (1 + 0.2 * torch.randn(head_dim, generator=g)).to(w_dtype)
    kw = (1 + 0.2 * torch.randn(head_dim, generator=g)).to(w_dtype)
    max_pos = 256
    cos = sin = None
    if rot:
        freqs = 1.0 / 10000.0 ** (torch.arange(0, rot, 2, dtype=torch.float64) / rot)
        angles = torch.arange(max_pos, dtype=torch.float64)[:, None] * freqs
        cos, sin = dev(angles.cos().float()), dev(angles.sin().float())
    positions = torch.tensor([p + t for p, n in zip(pasts, news) for t in range(n)], dtype=torch.int32)
    row_seq = torch.tensor([s for s, n in enumerate(news) for _ in range(n)], dtype=torch.int32)
    table = torch.tensor([[4, 5, 0], [7, 2, 0], [1, 8, 3]], dtype=torch.int32)
    assert K.qk_norm_rope_takes_sums(n_rows, head_dim, rot)
    results = []
    for source in (dev(rows), PartSums(dev(sums))):
        kp = torch.full((9, kv_heads, PAGE, head_dim), 768.0).to(torch.bfloat16)
        vp = torch.full((9, kv_heads, head_dim, PAGE), 768.0).to(torch.bfloat16)
        kp_d, vp_d = stored(K, kp, vp)
        q_out = torch.full((n_rows, n_heads * head_dim), 3.0, dtype=torch.bfloat16, device="cuda:0")
        K.qk_norm_rope_cache(source, q_out, dev(qw), dev(kw), 1e-5, cos, sin, dev(positions), dev(row_seq), kp_d, vp_d,
                             dev(table), n_heads, kv_heads, head_dim, True, int(positions.max()))
        results.append((q_out.cpu(), kp_d.cpu(), vp_d.cpu()))
    for from_rows, from_sums in zip(*results):
        assert torch.equal(from_rows, from_sums)
    assert not K.qk_norm_rope_takes_sums(63, head_dim, rot) and not K.qk_norm_rope_takes_sums(n_rows, 96, 96)
    with pytest.raises(Exception, match="sums in parts"):
        K.qk_norm_rope_cache(PartSums(dev(sums[:, :40].contiguous())), q_out[:40], dev(qw), dev(kw), 1e-5, cos, sin,
                             dev(positions[:40]), dev(row_seq[:40]), kp_d, vp_d, dev(table), n_heads, kv_heads, head_dim, True, 255)


@pytest.mark.parametrize("m,n,k", [(512, 6144, 4096), (1024, 6144, 4096), (333, 4080, 4096), (2048, 6144, 4096), (64, 6144, 4096),
                                   (640, 6144, 4096), (700, 6160, 2048)])        # two parts of the 192-wide tile
def test_product_left_in_parts_adds_up_to_the_finished_product(K, m, n, k):
    """`gemm_bare` leaves what `gemm` would have finished: the parts, added in their order and rounded, are its output bit
    for bit; where the library does not cut such a product it says so by returning None."""
    gen = torch.Generator().manual_seed(m + n)
    a = dev((torch.randn(m, k, generator=gen) * 0.5).to(torch.bfloat16))
    packed = K.pack_weight(dev((torch.randn(n, k, generator=gen) * 0.05).to(torch.bfloat16)))
    finished = torch.empty(m, n, dtype=torch.bfloat16, device="cuda:0")
    K.gemm(a, packed, finished)
    bare = K.gemm_bare(a, packed)
    if m in (2048, 64):           # a tile of its own, or few rows: not cut into parts for a finishing kernel of many rows
        assert bare is None
        return
    assert bare is not None and bare.parts >= 2 and tuple(bare.shape) == (m, n) and bare.dtype == torch.bfloat16
    total = torch.zeros(m, n, device="cuda:0")
    for part in range(bare.parts):
        total = total + bare.sums[part]
    assert torch.equal(total.to(torch.bfloat16), finished)
    assert K.gemm_bare(a.float(), packed) is None


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,width", [(1, 10), (7, 200), (33, 12288), (2, 25600)])
def test_swiglu(K, dtype, rows, width):
    g = torch.Generator().manual_seed(width)
    gu = (torch.randn(rows, 2 * width, generator=g) * 3).to(dtype)
    out = torch.empty(rows, width, dtype=dtype, device="cuda:0")
    K.swiglu(dev(gu), out)
    gate, up = gu[:, :width].double(), gu[:, width:].double()
    assert rel(out, gate / (1 + torch.exp(-gate)) * up) < tol(dtype, 2e-6, 4e-3)


@pytest.mark.parametrize("vocab", [7, 331, 1024, 1500, 8191, 8192, 8193, 10000, 151936])
def test_argmax_ties_go_to_the_lowest_id(K, vocab):
    g = torch.Generator().manual_seed(vocab)
    logits = torch.randn(5, vocab, generator=g)
    logits[1, vocab - 1] = 50.0
    logits[2, 0] = 50.0
    top = min(vocab - 1, 700)
    logits[3, top] = 60.0
    logits[3, top // 2] = 60.0               # a tie: the lower id wins
    logits[3, vocab - 1] = 60.0              # ... also against one far away (another chunk of a long row)
    logits[4, :] = 1.25                      # all equal: id 0
    tokens = torch.empty(5, dtype=torch.int32, device="cuda:0")
    bad = torch.empty(5, dtype=torch.int32, device="cuda:0")
    K.sample(dev(logits), tokens, bad)
    assert tokens.cpu().tolist() == [int(torch.argmax(logits[0])), vocab - 1, 0, top // 2, 0]
    assert bad.cpu().tolist() == [0] * 5


@pytest.mark.parametrize("vocab", [100, 20000])
def test_sample_flags_rows_that_are_not_finite(K, vocab):
    logits = torch.randn(3, vocab)
    logits[1, (2 * vocab) // 5] = float("nan")
    logits[2, vocab - 1] = float("inf")
    tokens = torch.empty(3, dtype=torch.int32, device="cuda:0")
    bad = torch.empty(3, dtype=torch.int32, device="cuda:0")
    K.sample(dev(logits), tokens, bad)
    assert bad.cpu().tolist() == [0, 1, 1] and tokens.cpu().tolist()[1:] == [-1, -1]


@pytest.mark.parametrize("vocab", [331, 2048, 151936])
def test_temperature_sampling_is_an_inverse_cdf_draw(K, vocab):
    g = torch.Generator().manual_seed(vocab)
    n = 64
    logits = torch.randn(n, vocab, generator=g) * 2
    temperature = torch.rand(n, generator=g) * 1.5 + 0.2
    uniform = torch.rand(n, generator=g)
    uniform[0], uniform[1] = 0.0, 0.99999994
    tokens = torch.empty(n, dtype=torch.int32, device="cuda:0")
    bad = torch.empty(n, dtype=torch.int32, device="cuda:0")
    K.sample(dev(logits), tokens, bad, temperature=dev(temperature), uniform=dev(uniform))
    probs = torch.softmax(logits.double() / temperature.double()[:, None], -1)
    cdf = torch.cumsum(probs, -1)
    for row, token in enumerate(tokens.cpu().tolist()):
        lower = float(cdf[row, token - 1]) if token > 0 else 0.0
        u = float(uniform[row])
        assert lower - 1e-5 <= u <= float(cdf[row, token]) + 1e-5, (row, token, lower, u, float(cdf[row, token]))
    # rows do not influence each other
    alone = torch.empty(1, dtype=torch.int32, device="cuda:0")
    K.sample(dev(logits[5:6]), alone, bad[:1].clone(), temperature=dev(temperature[5:6]), uniform=dev(uniform[5:6]))
    assert int(alone.cpu()) == int(tokens[5].cpu())


def test_top_k_and_top_p_restrict_the_draw(K):
    vocab, n = 1000, 200
    g = torch.Generator().manual_seed(3)
    logits = (torch.randn(1, vocab, generator=g) * 3).repeat(n, 1)
    uniform = torch.rand(n, generator=g)
    temperature = torch.ones(n)
    tokens = torch.empty(n, dtype=torch.int32, device="cuda:0")
    bad = torch.empty(n, dtype=torch.int32, device="cuda:0")
    top_k = torch.full((n,), 5, dtype=torch.int32)
    K.sample(dev(logits), tokens, bad, temperature=dev(temperature), top_k=dev(top_k), uniform=dev(uniform))
    allowed = set(torch.topk(logits[0], 5).indices.tolist())
    drawn = set(tokens.cpu().tolist())
    assert drawn <= allowed and len(drawn) > 1
    # top-p: the smallest set of most likely tokens whose mass reaches p
    p = 0.6
    probs = torch.softmax(logits[0].double(), 0)
    order = torch.argsort(probs, descending=True)
    count = int(torch.searchsorted(torch.cumsum(probs[order], 0), torch.tensor(p, dtype=torch.float64))) + 1
    nucleus = set(order[:count].tolist())
    K.sample(dev(logits), tokens, bad, temperature=dev(temperature), top_p=dev(torch.full((n,), p)), uniform=dev(uniform))
    drawn = set(tokens.cpu().tolist())
    assert drawn <= nucleus and len(drawn) > 1
    # k = 1 is greedy whatever the uniform number
    K.sample(dev(logits), tokens, bad, temperature=dev(temperature), top_k=dev(torch.ones(n, dtype=torch.int32)),
             uniform=dev(uniform))
    assert set(tokens.cpu().tolist()) == {int(torch.argmax(logits[0]))}


def test_kernels_refuse_what_they_cannot_do(K):
    from beholdd.kernels import KernelError
    x = torch.zeros(2, 8, device="cuda:0")
    with pytest.raises(KernelError):
        K.gemm(x, torch.zeros(4, 9, device="cuda:0"), torch.zeros(2, 4, device="cuda:0"))
    with pytest.raises(KernelError):
        K.gemm(x.cpu(), torch.zeros(4, 8, device="cuda:0"), torch.zeros(2, 4, device="cuda:0"))
    with pytest.raises(KernelError):
        K.rmsnorm(x, torch.ones(7, device="cuda:0"), 1e-6, torch.zeros(2, 8, device="cuda:0"))
    with pytest.raises(KernelError):      # a head size above the attention kernels' limit
        hd = 512
        K.attention(torch.zeros(1, hd, device="cuda:0"), torch.zeros(1, hd, device="cuda:0"),
                    torch.zeros(1, 1, PAGE, hd, device="cuda:0"), torch.zeros(1, 1, hd, PAGE, device="cuda:0"),
                    torch.zeros(1, 1, dtype=torch.int32, device="cuda:0"), torch.zeros(1, dtype=torch.int32, device="cuda:0"),
                    torch.zeros(1, dtype=torch.int32, device="cuda:0"), 1, 1, hd, 1.0)
