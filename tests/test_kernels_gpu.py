"""Each kernel alone against a plain float64 formula, at sizes other than the engine's."""
import math

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def rnd(*shape, seed=0, scale=1.0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g, dtype=torch.float64) * scale).to(dtype)


def to_dev(t, dtype=None):
    return t.to(device=DEV, dtype=dtype or t.dtype).contiguous()


# ----------------------------------------------------------------------- products
# (rows of W, k, tokens): the awkward shapes of the reference's own matmul test
# (crates/glassbox-core/src/kernels.rs:697) and larger ones that cross tile edges
GEMM_SHAPES_F32 = [(1, 32, 1), (8, 64, 2), (17, 64, 3), (33, 96, 9), (50, 160, 17), (331, 100, 70), (130, 257, 129),
                   # few rows through the skinny kernel: a k of one slice and a part, of many groups of slices, rows of W
                   # that do not fill the last workgroup, rows of A in several passes
                   (2048, 2048, 1), (50, 100, 5), (2048, 8192, 8), (331, 2120, 16), (96, 4100, 33), (1000, 72, 64),
                   (130, 258, 7)]
GEMM_SHAPES_BF16 = [(1, 32, 1), (8, 64, 2), (17, 64, 3), (33, 96, 9), (50, 160, 17), (331, 104, 64), (331, 104, 65),
                    (130, 264, 129), (16, 2048, 8), (272, 72, 300), (49, 520, 33),
                    # few rows of W and a long k: the skinny kernels split k over the waves of a workgroup
                    (2048, 2048, 8), (2048, 8192, 8), (64, 2056, 1), (100, 4104, 33), (2048, 2048, 64), (48, 8192, 17),
                    # the tiled kernel over many k-steps, k a multiple of its step and not, one and two
                    # k-steps of prefetch (few and many tiles), fewer k-steps than the prefetch reaches
                    (512, 1024, 200), (2048, 2048, 130), (96, 8192, 70), (1536, 1088, 520), (200, 128, 66), (3000, 192, 300),
                    (640, 1032, 257),
                    # a k of twelve to fifteen 64-wide blocks on sixteen waves (some of which find no block, or a part of one)
                    (960, 960, 12), (2560, 960, 33), (1600, 776, 20), (5120, 1016, 64)]


@pytest.mark.parametrize("N,K,M", GEMM_SHAPES_F32)
@pytest.mark.parametrize("accumulate", [False, True])
def test_gemm_f32(N, K, M, accumulate):
    from glassbox_amd import ops
    a, w, c0 = rnd(M, K, seed=1), rnd(N, K, seed=2), rnd(M, N, seed=3)
    want = a.double() @ w.double().T + (c0.double() if accumulate else 0)
    c = to_dev(c0.clone())
    ops.gemm(to_dev(a), to_dev(w), c, accumulate=accumulate)
    err = (c.cpu().double() - want).abs().max().item()
    assert err <= 1e-4 * (1 + want.abs().max().item()), err   # kernels.rs:716 tolerance


@pytest.mark.parametrize("N,K", [(1, 32), (50, 160), (17, 64), (331, 100), (96, 4100), (2048, 2048), (512, 8192), (8, 16384)])
def test_gemm_f32_is_summed_in_one_order_by_both_kernels_and_at_every_number_of_rows(N, K):
    """A cell's sum is cut into slices of 64 of k, each a chain of fused multiply-adds from zero, added in order
    (``csrc/hip/gemm_f32.hip``): the skinny kernel (8 rows of W a workgroup, a lane a slice) and the tiled one give the
    same bits, and a row of A gives the same bits alone, among 8 and among 70 rows, which is what lets batched
    and unbatched generation agree exactly in 32-bit."""
    from glassbox_amd import ops
    lib = ops._lib("gemm_f32")
    stream = torch.cuda.current_stream().cuda_stream
    a, w = to_dev(rnd(70, K, seed=5)), to_dev(rnd(N, K, seed=6))
    c0 = to_dev(rnd(70, N, seed=7))

    def run(rows, which, accumulate):
        c = c0[:rows].clone()
        rc = lib.gb_gemm_f32_by(a.data_ptr(), K, w.data_ptr(), K, c.data_ptr(), N, rows, N, K, accumulate, which, stream)
        assert rc == 0, lib.gb_last_error().decode()
        return c.cpu()

    for accumulate in (0, 1):
        tiled = run(70, 1, accumulate)
        want = a.cpu().double() @ w.cpu().double().T + (c0.cpu().double() if accumulate else 0)
        assert (tiled.double() - want).abs().max().item() <= 1e-4 * (1 + want.abs().max().item())
        for rows in (1, 2, 3, 8, 13, 16, 17, 40, 64):
            skinny = run(rows, 2, accumulate)
            assert torch.equal(skinny, tiled[:rows]), f"{rows} rows: the skinny kernel's bits differ from the tiled kernel's"
            assert torch.equal(run(rows, 1, accumulate), tiled[:rows]), f"{rows} rows: the tiled kernel's bits depend on M"
    # the skinny kernel is refused where it does not apply, not run wrongly
    assert lib.gb_gemm_f32_by(a.data_ptr(), K, w.data_ptr(), K, c0.data_ptr(), N, 70, N, K, 0, 2, stream) == 1
    assert "skinny" in lib.gb_last_error().decode()


@pytest.mark.parametrize("N,K,M", [(331, 100, 200), (130, 260, 129), (2048, 2048, 300), (512, 8192, 65), (96, 4100, 331),
                                   (257, 16, 128), (128, 72, 1)])
def test_gemm_f32_wide_kernel_gives_the_bits_of_the_tiled_kernel(N, K, M):
    """The kernel for prompts (128 x 64 of C a workgroup, 8 x 4 cells a thread, two k-steps in LDS) keeps the one
    summation order: the same bits as the tiled kernel, with and without accumulation, on tiles that hang over
    every edge; and it is refused where rows are no 16-byte words."""
    from glassbox_amd import ops
    lib = ops._lib("gemm_f32")
    stream = torch.cuda.current_stream().cuda_stream
    a, w, c0 = to_dev(rnd(M, K, seed=11)), to_dev(rnd(N, K, seed=12)), to_dev(rnd(M, N, seed=13))
    for accumulate in (0, 1):
        got = {}
        for which in (1, 3):
            c = c0.clone()
            rc = lib.gb_gemm_f32_by(a.data_ptr(), K, w.data_ptr(), K, c.data_ptr(), N, M, N, K, accumulate, which, stream)
            assert rc == 0, lib.gb_last_error().decode()
            got[which] = c.cpu()
        want = a.cpu().double() @ w.cpu().double().T + (c0.cpu().double() if accumulate else 0)
        assert (got[1].double() - want).abs().max().item() <= 1e-4 * (1 + want.abs().max().item())
        assert torch.equal(got[3], got[1]), "the wide kernel's bits differ from the tiled kernel's"
    if K > 4:
        assert lib.gb_gemm_f32_by(a.data_ptr() + 4, K, w.data_ptr(), K, c0.data_ptr(), N, M, N, K - 4, 0, 3, stream) == 1
        assert "wide" in lib.gb_last_error().decode()


def test_gemm_f32_takes_rows_that_are_no_words_of_16_bytes():
    """A k that is no multiple of 4, or operands that start in the middle of a word, go through the tiled kernel."""
    from glassbox_amd import ops
    for K, off in ((30, 0), (32, 1), (257, 0)):
        a, w = rnd(5, K + off, seed=8), rnd(20, K + off, seed=9)
        c = to_dev(torch.zeros(5, 20))
        da, dw = to_dev(a)[:, off:], to_dev(w)[:, off:]
        ops.gemm(da, dw, c)
        want = a[:, off:].double() @ w[:, off:].double().T
        assert (c.cpu().double() - want).abs().max().item() <= 1e-4 * (1 + want.abs().max().item())


@pytest.mark.parametrize("N,K,M", GEMM_SHAPES_BF16)
@pytest.mark.parametrize("out", ["bf16", "f32", "f32+"])
def test_gemm_bf16(N, K, M, out):
    from glassbox_amd import ops
    a, w = rnd(M, K, seed=1).bfloat16(), rnd(N, K, seed=2).bfloat16()
    c0 = rnd(M, N, seed=3)
    want = a.double() @ w.double().T + (c0.double() if out == "f32+" else 0)
    c = to_dev(c0.clone(), torch.bfloat16 if out == "bf16" else torch.float32)
    ops.gemm(to_dev(a), to_dev(w), c, accumulate=(out == "f32+"))
    got = c.cpu().double()
    # products of bfloat16 numbers are exact in 32-bit; only the summation order and (for a
    # bfloat16 result) the final rounding differ from the float64 sum
    tol = 1e-4 * math.sqrt(K) + (2 ** -8) * want.abs().max().item() * (out == "bf16")
    assert (got - want).abs().max().item() <= tol


@pytest.mark.parametrize("I,K,M", [(8, 32, 1), (176, 64, 5), (144, 80, 16), (200, 2048, 17), (8192, 2048, 8), (88, 4104, 64),
                                   # more than 64 rows: the tiled kernel's epilogue
                                   (176, 64, 130), (72, 264, 65), (1024, 520, 300), (2560, 960, 200), (2560, 960, 400), (1000, 2048, 129)])
def test_gemm_bf16_fused_silu_mul(I, K, M):
    """Stacked gate/up rows with the activation applied in the product's epilogue
    (crates/glassbox-core/src/model.rs:335-340), against the formula in float64."""
    from glassbox_amd import ops
    a, w = rnd(M, K, seed=1).bfloat16(), (rnd(2 * I, K, seed=2) / math.sqrt(K)).bfloat16()
    gu = a.double() @ w.double().T
    g, u = gu[:, :I], gu[:, I:]
    want = g / (1 + torch.exp(-g)) * u
    for dt in (torch.bfloat16, torch.float32):
        out = torch.full((M, I), 7.0, device=DEV, dtype=dt)
        ops.gemm(to_dev(a), to_dev(w), out, silu_mul=True)
        tol = 1e-4 + (2 ** -8) * want.abs().max().item() * (dt == torch.bfloat16)
        assert (out.cpu().double() - want).abs().max().item() <= tol
    # twice in a row: the same again
    out2 = torch.empty(M, I, device=DEV, dtype=torch.float32)
    ops.gemm(to_dev(a), to_dev(w), out2, silu_mul=True)
    assert torch.equal(out2, out)


@pytest.mark.parametrize("M,N,K", [(2100, 14000, 160), (1024, 28672, 128), (2048, 16384, 2048), (4000, 7200, 352),
                                   (2049, 14080, 128 + 32), (2048, 6144, 128),
                                   # 192 and 384 tiles, the last column tile partly outside
                                   (2048, 6000, 192), (4096, 6096, 160)])
@pytest.mark.parametrize("mode", ["bf16", "f32", "f32+", "silu"])
def test_gemm_bf16_large_products_through_the_lds_ring(M, N, K, mode):
    """Products of a thousand rows and more with some hundred 256 x 256 tiles take the kernel whose operands go
    from memory straight into a ring of LDS buffers: rows and columns that do not fill the last tiles, k-steps
    from the ring's depth upwards, every epilogue; twice in a row gives the same bits."""
    from glassbox_amd import ops
    a, w = rnd(M, K, seed=11).bfloat16(), rnd(N, K, seed=12).bfloat16()
    if mode == "silu":
        a, w = a * 0.25, w * 0.25
    full = a.double() @ w.double().T
    c0 = rnd(M, N, seed=13)
    if mode == "silu":
        g, u = full[:, :N // 2], full[:, N // 2:]
        want = g / (1 + torch.exp(-g)) * u
    else:
        want = full + (c0.double() if mode == "f32+" else 0)
    outs = []
    for _ in range(2):
        if mode == "silu":
            c = torch.full((M, N // 2), 7.0, device=DEV, dtype=torch.bfloat16)
        else:
            c = to_dev(c0.clone(), torch.bfloat16 if mode == "bf16" else torch.float32)
        ops.gemm(to_dev(a), to_dev(w), c, accumulate=(mode == "f32+"), silu_mul=(mode == "silu"))
        outs.append(c)
    tol = 1e-4 * math.sqrt(K) + (2 ** -8) * want.abs().max().item() * (mode in ("bf16", "silu"))
    assert (outs[0].cpu().double() - want).abs().max().item() <= tol
    assert torch.equal(outs[0], outs[1])


@pytest.mark.parametrize("N,K,M,silu", [(96, 64, 1, False), (6144, 2048, 8, False), (352, 176, 5, True),
                                        (16384, 2048, 8, True), (480, 80, 33, False), (512, 4104, 64, True)])
@pytest.mark.parametrize("gamma_dtype", [torch.float32, torch.bfloat16])
def test_gemm_bf16_fused_rms_norm(N, K, M, silu, gamma_dtype):
    """The product that norms its float32 rows on the way, against norm-then-product in float64
    (crates/glassbox-core/src/model.rs:94-100 and 260 / 335)."""
    from glassbox_amd import ops
    x = rnd(M, K, seed=1, scale=3.0).float()
    x[0] *= 1e-3                                              # a row where eps matters
    g = (rnd(K, seed=2) * 0.3 + 1.0).to(gamma_dtype)
    w = (rnd(N, K, seed=3) / math.sqrt(K)).bfloat16()
    eps = 1e-5
    h = g.double() * (x.double() * torch.rsqrt(x.double().pow(2).mean(-1, keepdim=True) + eps))
    prod = h @ w.double().T
    if silu:
        gate, up = prod[:, :N // 2], prod[:, N // 2:]
        want = gate / (1 + torch.exp(-gate)) * up
    else:
        want = prod
    out = torch.full(want.shape, 9.0, device=DEV, dtype=torch.bfloat16)
    ops.gemm(to_dev(x), to_dev(w), out, silu_mul=silu, rms=(to_dev(g), eps))
    # bf16(g * x) as the operand: one rounding per element, 2^-9 relative, averaged over k
    tol = (2 ** -7) * want.abs().max().item() + 1e-3
    assert (out.cpu().double() - want).abs().max().item() <= tol
    # the unfused pair of kernels rounds elsewhere (bf16(g * x * s) as the operand) and is as close
    hn = torch.empty(M, K, device=DEV, dtype=torch.bfloat16)
    ops.rmsnorm(to_dev(x), to_dev(g), eps, hn)
    two = torch.empty_like(out)
    ops.gemm(hn, to_dev(w), two, silu_mul=silu)
    assert (two.cpu().double() - want).abs().max().item() <= tol


@pytest.mark.parametrize("M,N,K,N2,silu", [(1, 64, 176, 96, False), (5, 352, 64, 176, True), (8, 2048, 2048, 6144, False),
                                           (8, 2048, 8192, 16384, True), (3, 960, 2560, 2880, False),
                                           # more than 8 rows: the skinny kernel emits (tiles of 8 columns while they are
                                           # few, of 16 beyond), and takes the partial sums of up to 64 rows
                                           (12, 960, 2560, 2880, False), (40, 24704, 128, 512, False), (64, 352, 64, 176, True),
                                           (20, 4096, 1024, 1024, True), (9, 72, 264, 48, False), (17, 2048, 1024, 16384, True),
                                           (20, 960, 960, 5120, True), (33, 960, 776, 1600, False),
                                           # at most 8 rows by so many rows of W that the folded kernel does not pay
                                           (5, 4096, 512, 256, False)])
@pytest.mark.parametrize("gamma_dtype", [torch.float32, torch.bfloat16])
def test_gemm_bf16_prepares_the_next_norm(M, N, K, N2, silu, gamma_dtype):
    """The product that adds into the residual and, on its way out, writes what the RMS norm that reads
    the residual next would compute (bf16(gamma * r) and partial sums of r^2), and the product that takes
    those: against norm-then-product in float64 (crates/glassbox-core/src/model.rs:94-100, 323-335)."""
    from glassbox_amd import ops
    parts_n = ops.gemm_emit_parts(M, N)
    assert parts_n == (-(-N // 8) if -(-N // 16) < 256 else -(-N // 16)) and ops.gemm_emit_mode(M, N, K) == 1
    stride = ops.parts_stride(M)
    assert stride == (8 if M <= 8 else 64)
    a, w = rnd(M, K, seed=1).bfloat16(), (rnd(N, K, seed=2) / math.sqrt(K)).bfloat16()
    r0 = rnd(M, N, seed=3, scale=2.0).float()
    g = (rnd(N, seed=4) * 0.3 + 1.0).to(gamma_dtype)
    eps = 1e-5
    plain = to_dev(r0.clone())
    ops.gemm(to_dev(a), to_dev(w), plain, accumulate=True)
    res, h = to_dev(r0.clone()), torch.zeros(M, N, device=DEV, dtype=torch.bfloat16)
    parts = torch.full((parts_n, stride), 7.0, device=DEV)
    ops.gemm(to_dev(a), to_dev(w), res, accumulate=True, emit=(to_dev(g), h, parts))
    assert torch.equal(res, plain)                                        # the residual is what it was without
    assert torch.equal(h, (to_dev(g).float() * res).bfloat16())
    ss = res.double().pow(2).sum(-1).cpu()
    assert ((parts[:, :M].double().sum(0).cpu() - ss).abs() <= 1e-5 * ss).all()
    assert ((parts[:, M:] == 0) | (parts[:, M:] == 7.0)).all()                # rows that do not exist: zero or untouched
    # the product that follows
    w2 = (rnd(N2, N, seed=5) / math.sqrt(N)).bfloat16()
    x = res.double().cpu()
    normed = g.double() * (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps))
    prod = normed @ w2.double().T
    want = prod if not silu else prod[:, :N2 // 2] / (1 + torch.exp(-prod[:, :N2 // 2])) * prod[:, N2 // 2:]
    out = torch.full(want.shape, 9.0, device=DEV, dtype=torch.bfloat16)
    ops.gemm(h, to_dev(w2), out, silu_mul=silu, rms_parts=(parts, parts_n, eps))
    tol = (2 ** -7) * want.abs().max().item() + 1e-3                      # as for the norm computed on the way in
    assert (out.cpu().double() - want).abs().max().item() <= tol
    again = torch.empty_like(out)
    ops.gemm(res, to_dev(w2), again, silu_mul=silu, rms=(to_dev(g), eps))
    assert ((out.float() - again.float()).abs() <= 2 ** -6 * (1 + again.float().abs())).all()


@pytest.mark.parametrize("M,N,K", [(2048, 2048, 8192), (128, 2048, 2048), (40, 1008, 4104), (300, 960, 2560), (64, 2048, 8192)])
@pytest.mark.parametrize("gamma_dtype", [torch.float32, torch.bfloat16])
def test_gemm_bf16_that_divides_k_does_the_next_norm(M, N, K, gamma_dtype):
    """An accumulating product that divides k over workgroups adds its slices row by row, and with a row in hand
    writes the RMS norm of the new residual too: the rows the norm's own kernel would give."""
    from glassbox_amd import ops
    assert ops.gemm_emit_mode(M, N, K) == 2 and ops.gemm_emit_mode(4, N, K) != 2
    a, w = (rnd(M, K, seed=21) * 0.5).bfloat16(), (rnd(N, K, seed=22) * 0.1).bfloat16()
    res0, g = rnd(M, N, seed=23).float(), (rnd(N, seed=24) * 0.3 + 1).to(gamma_dtype)
    eps = 1e-5
    ws = torch.empty(ops.gemm_split_floats(M, N, K), device=DEV)
    res, h = to_dev(res0.clone()), torch.full((M, N), 9.0, device=DEV, dtype=torch.bfloat16)
    ops.gemm(to_dev(a), to_dev(w), res, accumulate=True, emit=(to_dev(g), h, eps), workspace=ws)
    want_res = res0.double() + a.double() @ w.double().T
    assert (res.cpu().double() - want_res).abs().max().item() <= 1e-4 * math.sqrt(K)
    # the residual is the same as without the norm, bit for bit; the rows are those of the norm's kernel but for
    # the order of its sum (a unit in the last place of bfloat16 at most)
    plain = to_dev(res0.clone())
    ops.gemm(to_dev(a), to_dev(w), plain, accumulate=True, workspace=ws)
    assert torch.equal(res, plain)
    normed = torch.empty_like(h)
    ops.rmsnorm(res, to_dev(g), eps, normed)
    assert ((h.float() - normed.float()).abs() <= 2 ** -7 * normed.float().abs() + 1e-6).all()
    x = res.cpu().double()
    want = g.double() * x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    assert (h.cpu().double() - want).abs().max().item() <= 2 ** -8 * want.abs().max().item() + 1e-6
    with pytest.raises(ops.KernelError, match="norm"):
        ops.gemm(to_dev(a), to_dev(w), res, accumulate=True, emit=(to_dev(g), h, eps))       # no workspace


@pytest.mark.parametrize("M,N,K", [(17, 96, 4096), (33, 2048, 2048), (64, 2048, 8192), (100, 2048, 4160),
                                   # 128 narrow tiles are not enough to go without slices (Llama-3-8B's O and down projections)
                                   (96, 4096, 8192), (128, 4096, 4096),
                                   # beyond 64 rows a slice of a long k keeps 1,024 of it
                                   (192, 2048, 4096), (256, 1024, 8192),
                                   # a k that is no multiple of 64: the tiled kernel's slices
                                   (200, 528, 8200), (40, 1008, 4104),
                                   # a thousand rows and more: slices of k through the 256 x 256 tiles
                                   (2048, 2048, 8192), (1100, 1008, 4160), (1024, 528, 5120),
                                   # some hundred rows, a k of 2,048 and very few tiles
                                   (128, 2048, 2048), (300, 1008, 2112), (256, 1024, 2048)])
@pytest.mark.parametrize("mode", ["bf16", "f32", "f32+", "silu"])
def test_gemm_bf16_divides_k_over_workgroups(M, N, K, mode):
    """With a workspace, a product of few tiles has several workgroups a tile, each over a slice of k,
    and a second kernel adds their sums in a fixed order and applies the epilogue: against float64, and
    the same bits on every run."""
    from glassbox_amd import ops
    floats = ops.gemm_split_floats(M, N, K)
    assert floats > 0 and floats % (M * N) == 0 and floats // (M * N) >= 2
    a, w = rnd(M, K, seed=1).bfloat16(), (rnd(N, K, seed=2) / math.sqrt(K)).bfloat16()
    c0 = rnd(M, N, seed=3)
    prod = a.double() @ w.double().T
    if mode == "silu":
        want = prod[:, :N // 2] / (1 + torch.exp(-prod[:, :N // 2])) * prod[:, N // 2:]
    else:
        want = prod + (c0.double() if mode == "f32+" else 0)
    ws = torch.full((floats + 3,), float("nan"), device=DEV)[:floats]
    outs = []
    for _ in range(2):
        if mode == "silu":
            c = torch.full((M, N // 2), 7.0, device=DEV, dtype=torch.bfloat16)
        else:
            c = to_dev(c0.clone(), torch.bfloat16 if mode == "bf16" else torch.float32)
        ops.gemm(to_dev(a), to_dev(w), c, accumulate=(mode == "f32+"), silu_mul=(mode == "silu"), workspace=ws)
        outs.append(c)
    tol = 1e-4 * math.sqrt(K) + (2 ** -8) * want.abs().max().item() * (mode in ("bf16", "silu"))
    assert (outs[0].cpu().double() - want).abs().max().item() <= tol
    assert torch.equal(outs[0], outs[1])
    with pytest.raises(ops.KernelError, match="workspace"):
        ops.gemm(to_dev(a), to_dev(w), outs[0], accumulate=(mode == "f32+"), silu_mul=(mode == "silu"), workspace=ws[:8])


@pytest.mark.parametrize("M,N,K", [(65, 6144, 2048), (128, 16384, 2048), (96, 6144, 8192),
                                   # one, two, three k-steps: fewer than either ring is deep; and more than both
                                   (100, 4096, 64), (128, 4128, 128), (100, 5000, 192), (70, 6200, 1024), (128, 8200, 1088),
                                   # so many narrow tiles that a workgroup takes 64 columns
                                   (128, 24600, 320), (96, 32760, 512),
                                   # 17 to 64 rows by very many rows of W: the wide tiles, not the skinny kernel
                                   (64, 49152, 256), (40, 33000, 192), (20, 40000, 192),
                                   # a narrow model's products: few narrow tiles and a k too short to divide; and up to
                                   # 256 rows (two row tiles) where the wide tiles would be fewer still
                                   (96, 2560, 960), (200, 5120, 960), (256, 2500, 448), (129, 2100, 128)])
@pytest.mark.parametrize("mode", ["bf16", "f32", "f32+", "silu"])
def test_gemm_bf16_streams_products_of_some_hundred_rows(M, N, K, mode):
    """65 to 128 rows (to 256 in a narrow model), a k that is a multiple of 64: tiles of 128 rows by 32 or 64 columns, both operands through
    rings in LDS, no slices of k where the narrow tiles alone fill the chip (with or without a workspace on offer).
    Against float64, the same bits on every run, rows and columns beyond the last tile's edge untouched."""
    from glassbox_amd import ops
    if mode == "silu" and N % 16:
        N -= N % 16
    assert ops.gemm_split_floats(M, N, K) == 0
    a, w = rnd(M, K, seed=1).bfloat16(), (rnd(N, K, seed=2) / math.sqrt(K)).bfloat16()
    c0 = rnd(M, N, seed=3)
    prod = a.double() @ w.double().T
    if mode == "silu":
        want = prod[:, :N // 2] / (1 + torch.exp(-prod[:, :N // 2])) * prod[:, N // 2:]
    else:
        want = prod + (c0.double() if mode == "f32+" else 0)
    cols = want.shape[1]
    outs = []
    for _ in range(2):
        # a frame of untouched cells around the result: two more rows, a longer row stride
        dtype = torch.float32 if mode in ("f32", "f32+") else torch.bfloat16
        frame = torch.full((M + 2, cols + 8), 7.0, device=DEV, dtype=dtype)
        c = frame[:M, :cols]
        if mode == "f32+":
            c.copy_(to_dev(c0))
        ops.gemm(to_dev(a), to_dev(w), c, accumulate=(mode == "f32+"), silu_mul=(mode == "silu"))
        assert (frame[M:] == 7.0).all() and (frame[:, cols:] == 7.0).all()
        outs.append(c.clone())
    tol = 1e-4 * math.sqrt(K) + (2 ** -8) * want.abs().max().item() * (mode in ("bf16", "silu"))
    assert (outs[0].cpu().double() - want).abs().max().item() <= tol
    assert torch.equal(outs[0], outs[1])


def test_gemm_bf16_split_k_is_the_same_on_every_run():
    from glassbox_amd import ops
    a, w = to_dev(rnd(8, 8192, seed=1).bfloat16()), to_dev(rnd(2048, 8192, seed=2).bfloat16())
    base = torch.zeros(8, 2048, device=DEV)
    ops.gemm(a, w, base, accumulate=True)
    for _ in range(5):
        again = torch.zeros(8, 2048, device=DEV)
        ops.gemm(a, w, again, accumulate=True)
        assert torch.equal(again, base)


def test_gemm_bf16_one_hot_rows_and_columns():
    """Every (row, column, k) lands where it should: W picks single columns of A."""
    from glassbox_amd import ops
    M, K, N = 150, 136, 200
    a = rnd(M, K, seed=5).bfloat16()
    w = torch.zeros(N, K)
    for n in range(N):
        w[n, (7 * n + 3) % K] = 1.0
    c = torch.zeros(M, N, device=DEV)
    ops.gemm(to_dev(a), to_dev(w.bfloat16()), c)
    want = a.float()[:, [(7 * n + 3) % K for n in range(N)]]
    assert torch.equal(c.cpu(), want)
    for rows in (9, 8, 5, 1):   # the skinny kernel, and the one that folds two k ranges into a tile
        c2 = torch.zeros(rows, N, device=DEV)
        ops.gemm(to_dev(a[:rows]), to_dev(w.bfloat16()), c2)
        assert torch.equal(c2.cpu(), want[:rows]), rows


def test_gemm_refuses_bad_inner_size():
    from glassbox_amd import ops
    a, w = torch.zeros(4, 12, device=DEV, dtype=torch.bfloat16), torch.zeros(8, 12, device=DEV, dtype=torch.bfloat16)
    with pytest.raises(ops.KernelError, match="multiple of 8"):
        ops.gemm(a, w, torch.zeros(4, 8, device=DEV, dtype=torch.bfloat16))


# -------------------------------------------------------------------- elementwise
@pytest.mark.parametrize("n,d", [(1, 7), (3, 100), (5, 576), (2, 1537), (4, 2048)])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_rmsnorm(n, d, out_dtype):
    from glassbox_amd import ops
    x, g, eps = rnd(n, d, seed=1, scale=3.0), rnd(d, seed=2) + 1.0, 3e-5
    want = g.double() * (x.double() * torch.rsqrt(x.double().pow(2).mean(-1, keepdim=True) + eps))
    out = torch.empty(n, d, device=DEV, dtype=out_dtype)
    ops.rmsnorm(to_dev(x), to_dev(g), eps, out)
    tol = 1e-5 if out_dtype == torch.float32 else 2 ** -8
    assert ((out.cpu().double() - want).abs() <= tol * (1 + want.abs())).all()
    # picked rows
    rows = torch.tensor([n - 1, 0], dtype=torch.int32, device=DEV)
    out2 = torch.empty(2, d, device=DEV, dtype=out_dtype)
    ops.rmsnorm(to_dev(x), to_dev(g), eps, out2, rows)
    assert torch.equal(out2.cpu(), out.cpu()[[n - 1, 0]])


def test_embed():
    from glassbox_amd import ops
    table = rnd(37, 50, seed=1)
    ids = torch.tensor([5, 0, 36, 5], dtype=torch.int32, device=DEV)
    for dt in (torch.float32, torch.bfloat16):
        out = torch.empty(4, 50, device=DEV)
        ops.embed(to_dev(table, dt), ids, out)
        assert torch.equal(out.cpu(), table.to(dt).float()[[5, 0, 36, 5]])


def test_silu_mul():
    from glassbox_amd import ops
    gu = rnd(6, 2 * 173, seed=4, scale=4.0)
    g, u = gu[:, :173].double(), gu[:, 173:].double()
    want = g / (1 + torch.exp(-g)) * u
    out = torch.empty(6, 173, device=DEV)
    ops.silu_mul(to_dev(gu), out)
    assert (out.cpu().double() - want).abs().max().item() < 1e-5


@pytest.mark.parametrize("hd,theta", [(16, 10000.0), (48, 500000.0), (128, 130000.0), (80, 10000.0),
                                      (10, 10000.0)])   # 10: no multiple of 4, the kernel that goes pair by pair
def test_rope_table_and_rotation(hd, theta):
    """Against the plain implementation: pairing (i, i + hd/2), sign, 32-bit angle at long positions."""
    from glassbox_amd import ops
    from glassbox_amd.parts.rotary import Rotary
    from plain import llama
    pos = [0, 1, 17, 4095, 100003]
    n, nh, nkv = len(pos), 3, 2
    rot = Rotary(hd, theta)
    cos = torch.empty(n, hd // 2, device=DEV)
    sin = torch.empty_like(cos)
    ops.rope_table(torch.tensor(pos, dtype=torch.int32, device=DEV), torch.from_numpy(rot.inv_host).to(DEV), cos, sin)
    s_want, c_want = llama.rope_angles(pos, hd, theta)
    assert np.abs(cos.cpu().numpy() - c_want).max() < 1e-7 and np.abs(sin.cpu().numpy() - s_want).max() < 1e-7
    qkv = rnd(n, (nh + 2 * nkv) * hd, seed=3)
    page = 16
    k_pages = torch.zeros(ops.key_pages_shape(4, nkv, page, hd), device=DEV)
    v_pages = torch.zeros(4, nkv, hd, page, device=DEV)
    slots = torch.tensor([3, 16 + 15, 32, 0, 63], dtype=torch.int32, device=DEV)
    buf = to_dev(qkv.clone())
    ops.rope_store(buf, cos, sin, slots, k_pages, v_pages, nh, nkv, hd)
    q_want = llama.rope(qkv[:, :nh * hd].double().reshape(n, nh, hd), pos, theta)
    k_want = llama.rope(qkv[:, nh * hd:(nh + nkv) * hd].double().reshape(n, nkv, hd), pos, theta)
    got_q = buf.cpu()[:, :nh * hd].double().reshape(n, nh, hd)
    assert (got_q - q_want).abs().max().item() < 1e-5
    assert torch.equal(got_q[0], qkv[0, :nh * hd].double().reshape(nh, hd)), "position 0 must leave the vector as it is"
    for i, s in enumerate(slots.tolist()):
        got_k = ops.unpack_keys(k_pages)[s // page, :, s % page, :].cpu().double()
        got_v = v_pages[s // page, :, :, s % page].cpu()
        assert (got_k - k_want[i]).abs().max().item() < 1e-5
        assert torch.equal(got_v, qkv[i, (nh + nkv) * hd:].reshape(nkv, hd))


ROPE_PRODUCTS = [(1, 4, 2, 16, 64), (8, 3, 1, 32, 96), (5, 6, 2, 48, 80), (8, 32, 32, 64, 2048), (33, 8, 2, 128, 264),
                 (64, 15, 5, 64, 960), (7, 4, 0, 32, 64),
                 # 432 and 400 tiles of 8 pairs: a tile and a half to a workgroup, and two tiles each
                 (40, 50, 2, 128, 128), (20, 48, 1, 128, 192)]


@pytest.mark.parametrize("nh,nkv,hd,page", [(4, 2, 16, 16), (32, 32, 64, 16), (5, 1, 48, 32), (8, 2, 128, 16), (3, 3, 80, 64)])
def test_rope_store_in_bfloat16_moves_whole_pieces(nh, nkv, hd, page):
    """bfloat16 rows of head sizes in steps of 16 (a lane takes 8 dimensions and their partners): rotated queries
    in the row, rotated keys in the row and in their pages, values in theirs, against float64
    (crates/glassbox-core/src/model.rs:102-115, 273-275)."""
    from glassbox_amd import ops
    from plain import llama
    n, theta = 37, 130000.0
    g = torch.Generator().manual_seed(hd)
    pos = torch.randint(0, 6000, (n,), generator=g).tolist()
    s64, c64 = llama.rope_angles(pos, hd, theta)
    cos, sin = to_dev(torch.from_numpy(c64).float()), to_dev(torch.from_numpy(s64).float())
    qkv = rnd(n, (nh + 2 * nkv) * hd, seed=7).bfloat16()
    pages = 4
    slots = torch.randperm(pages * page, generator=g)[:n].to(torch.int32)
    k_pages = torch.zeros(ops.key_pages_shape(pages, nkv, page, hd), device=DEV, dtype=torch.bfloat16)
    v_pages = torch.zeros(pages, nkv, hd, page, device=DEV, dtype=torch.bfloat16)
    buf = to_dev(qkv.clone())
    ops.rope_store(buf, cos, sin, to_dev(slots), k_pages, v_pages, nh, nkv, hd)
    q_want = llama.rope(qkv[:, :nh * hd].double().reshape(n, nh, hd), pos, theta)
    k_want = llama.rope(qkv[:, nh * hd:(nh + nkv) * hd].double().reshape(n, nkv, hd), pos, theta)
    got = buf.cpu()
    tol = 2 ** -8 * 1.5 * qkv.abs().max().item()   # one rounding to bfloat16 of a value up to sqrt(2) times the largest input
    assert (got[:, :nh * hd].double().reshape(n, nh, hd) - q_want).abs().max().item() <= tol
    assert (got[:, nh * hd:(nh + nkv) * hd].double().reshape(n, nkv, hd) - k_want).abs().max().item() <= tol
    assert torch.equal(got[:, (nh + nkv) * hd:], qkv[:, (nh + nkv) * hd:]), "values stay as they are"
    idx = slots.long()
    assert torch.equal(ops.unpack_keys(k_pages).cpu()[idx // page, :, idx % page, :], got[:, nh * hd:(nh + nkv) * hd].reshape(n, nkv, hd))
    assert torch.equal(v_pages.cpu()[idx // page, :, :, idx % page], qkv[:, (nh + nkv) * hd:].reshape(n, nkv, hd))
    free = torch.ones(pages * page, dtype=torch.bool)
    free[idx] = False
    fi = torch.nonzero(free).flatten()
    assert ops.unpack_keys(k_pages).cpu()[fi // page, :, fi % page, :].abs().sum().item() == 0
    assert v_pages.cpu()[fi // page, :, :, fi % page].abs().sum().item() == 0


@pytest.mark.parametrize("M,nh,nkv,hd,K,normed", [p + (False,) for p in ROPE_PRODUCTS] +
                         [p + (True,) for p in ROPE_PRODUCTS if p[0] <= 16])   # the norm on the way in serves 16 rows
def test_gemm_bf16_rotates_and_writes_the_cache(M, nh, nkv, hd, K, normed):
    """The stacked q/k/v product whose epilogue rotates query and key heads and writes keys and values into
    the pages: against the product, the rotation and the cache write in float64
    (crates/glassbox-core/src/model.rs:260-276), and against the two kernels it replaces."""
    from glassbox_amd import ops
    from plain import llama
    page, N = 16, (nh + 2 * nkv) * hd
    g = torch.Generator().manual_seed(M + hd)
    x = rnd(M, K, seed=1, scale=2.0).float()
    gamma, eps = (rnd(K, seed=2) * 0.3 + 1.0).float(), 1e-5
    w = (rnd(N, K, seed=3) / math.sqrt(K)).bfloat16()
    pos = torch.randint(0, 5000, (M,), generator=g).tolist()
    theta = 130000.0
    s64, c64 = llama.rope_angles(pos, hd, theta)
    cos, sin = to_dev(torch.from_numpy(c64).float()), to_dev(torch.from_numpy(s64).float())
    slots = torch.randperm(4 * page, generator=g)[:M].to(torch.int32)
    if normed:
        a_dev = to_dev(x)
        h64 = gamma.double() * (x.double() * torch.rsqrt(x.double().pow(2).mean(-1, keepdim=True) + eps))
        rms = (to_dev(gamma), eps)
    else:
        a_dev = to_dev(x.bfloat16())
        h64 = x.bfloat16().double()
        rms = None
    prod = h64 @ w.double().T
    q_want = llama.rope(prod[:, :nh * hd].reshape(M, nh, hd), pos, theta).reshape(M, nh * hd)
    store = nkv > 0
    k_pages = torch.zeros(ops.key_pages_shape(4, max(nkv, 1), page, hd), device=DEV, dtype=torch.bfloat16)
    v_pages = torch.zeros(4, max(nkv, 1), hd, page, device=DEV, dtype=torch.bfloat16)
    qkv = torch.full((M, N), 9.0, device=DEV, dtype=torch.bfloat16)
    ops.gemm_rope(a_dev, to_dev(w), qkv, nh, nkv, hd, cos, sin, to_dev(slots) if store else None,
                  k_pages if store else None, v_pages if store else None, rms=rms)
    tol = (2 ** -7) * prod.abs().max().item() + 1e-3
    assert (qkv[:, :nh * hd].cpu().double() - q_want).abs().max().item() <= tol
    if store:
        k_want = llama.rope(prod[:, nh * hd:(nh + nkv) * hd].reshape(M, nkv, hd), pos, theta)
        v_want = prod[:, (nh + nkv) * hd:].reshape(M, nkv, hd)
        for i, sl in enumerate(slots.tolist()):
            assert (ops.unpack_keys(k_pages)[sl // page, :, sl % page, :].cpu().double() - k_want[i]).abs().max().item() <= tol
            assert (v_pages[sl // page, :, :, sl % page].cpu().double() - v_want[i]).abs().max().item() <= tol
        # the rows hold what the pages hold
        assert torch.equal(qkv[0, nh * hd:(nh + nkv) * hd].reshape(nkv, hd),
                           ops.unpack_keys(k_pages)[slots[0] // page, :, slots[0] % page, :])
        # the two kernels it replaces round once more (the product to bfloat16 before the rotation)
        two = torch.empty_like(qkv)
        ops.gemm(a_dev, to_dev(w), two, rms=rms)
        k2, v2 = torch.zeros_like(k_pages), torch.zeros_like(v_pages)
        ops.rope_store(two, cos, sin, to_dev(slots), k2, v2, nh, nkv, hd)
        # (a rotated value can be much smaller than the two it is made of, so the bound is absolute)
        assert (two.float() - qkv.float()).abs().max().item() <= 2 * tol
        assert (k2.float() - k_pages.float()).abs().max().item() <= 2 * tol
        assert (v2.float() - v_pages.float()).abs().max().item() <= 2 * tol


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hd,page", [(16, 16), (64, 16), (128, 32), (40, 16)])
def test_rope_store_writes_values_of_portions_in_tiles(dtype, hd, page):
    """Values of prompt portions go to the transposed pages sixteen positions at a time: the pages must
    come out as when every row is written by itself.  Portions that start in the middle of a page, end
    in the middle of one, are shorter than a page, and single rows before them."""
    from glassbox_amd import ops
    nh, nkv = 3, 2
    q_lens, pos0 = [1, 1, 40, 16, 7, 33], [9, 0, 5, 32, 0, 47]
    n, n_dec = sum(q_lens), 2
    q_start = np.concatenate([[0], np.cumsum(q_lens)[:-1]]).tolist()
    pages_of, slots, next_page = [], [], 0
    for length, first in zip(q_lens, pos0):                   # every request has pages of its own, in a scrambled order
        count = -(-(first + length) // page)
        mine = [next_page + (7 * i) % count for i in range(count)] if count % 7 else list(range(next_page, next_page + count))
        next_page += count
        pages_of.append(mine)
        slots += [mine[p // page] * page + p % page for p in range(first, first + length)]
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    qkv = rnd(n, (nh + 2 * nkv) * hd, seed=5).to(dtype)
    cos, sin = torch.rand(n, hd // 2, device=DEV), torch.rand(n, hd // 2, device=DEV)
    results = []
    for portions in (None, (n_dec, i32(q_start), i32(q_lens), i32(pos0), n_dec, len(q_lens) - n_dec, max(q_lens))):
        k_pages = torch.zeros(ops.key_pages_shape(next_page, nkv, page, hd), device=DEV, dtype=dtype)
        v_pages = torch.zeros(next_page, nkv, hd, page, device=DEV, dtype=dtype)
        buf = to_dev(qkv.clone())
        ops.rope_store(buf, cos, sin, i32(slots), k_pages, v_pages, nh, nkv, hd, portions=portions)
        results.append((buf.cpu(), k_pages.cpu(), v_pages.cpu()))
    for a, b in zip(*results):
        assert torch.equal(a, b)
    assert results[0][2].abs().sum() > 0


# ---------------------------------------------------------------------- attention
def paged_setup(ctx_lens, nkv, hd, page, seed, dtype, scatter=True):
    """Keys and values of several requests scattered over pages in a shuffled order."""
    g = torch.Generator().manual_seed(seed)
    total_pages = sum(-(-c // page) for c in ctx_lens) + 3
    perm = torch.randperm(total_pages, generator=g).tolist() if scatter else list(range(total_pages))
    k_pages = torch.randn(total_pages, nkv, page, hd, generator=g).to(dtype)   # unowned slots hold junk
    v_pages = torch.randn(total_pages, nkv, hd, page, generator=g).to(dtype)   # values are kept transposed
    tables, ks, vs = [], [], []
    for c in ctx_lens:
        np_ = -(-c // page)
        t = [perm.pop() for _ in range(np_)]
        tables.append(t)
        k = torch.randn(c, nkv, hd, generator=g).to(dtype)
        v = torch.randn(c, nkv, hd, generator=g).to(dtype)
        for p in range(c):
            k_pages[t[p // page], :, p % page, :] = k[p]
            v_pages[t[p // page], :, :, p % page] = v[p]
        ks.append(k)
        vs.append(v)
    maxp = max(len(t) for t in tables)
    table_t = torch.tensor([t + [-1] * (maxp - len(t)) for t in tables], dtype=torch.int32)
    return k_pages, v_pages, table_t, ks, vs


def plain_attention_rows(q, ks, vs, tok_seq, positions, nh, scale, window):
    out = torch.zeros_like(q, dtype=torch.float64)
    n, _ = q.shape
    hd = ks[0].shape[-1]
    group = nh // ks[0].shape[1]
    for i in range(n):
        k, v, p = ks[tok_seq[i]].double(), vs[tok_seq[i]].double(), positions[i]
        lo = max(0, p - window + 1) if window else 0
        for h in range(nh):
            s = (k[lo:p + 1, h // group] @ q[i, h * hd:(h + 1) * hd].double()) * scale
            w = torch.softmax(s, 0)
            out[i, h * hd:(h + 1) * hd] = w @ v[lo:p + 1, h // group]
    return out


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,nkv,hd,window", [(4, 2, 16, 0), (3, 1, 32, 0), (6, 2, 48, 0), (8, 8, 64, 0),
                                              (8, 2, 128, 0), (5, 5, 80, 0), (4, 2, 32, 37), (2, 1, 256, 0)])
def test_attention_plain_kernel(dtype, nh, nkv, hd, window):
    from glassbox_amd import ops
    page = 16
    ctx_lens = [1, 300, 77, 16, 530]
    k_pages, v_pages, tables, ks, vs = paged_setup(ctx_lens, nkv, hd, page, seed=hd + nh, dtype=dtype)
    # rows: the last token of every request, plus a portion in the middle of request 1 and the first tokens of 4
    tok_seq = [0, 1, 2, 3, 4] + [1] * 5 + [4] * 3
    positions = [c - 1 for c in ctx_lens] + [100, 101, 102, 103, 104] + [0, 1, 2]
    n = len(tok_seq)
    q = rnd(n, nh * hd, seed=11).to(dtype)
    scale = 1 / math.sqrt(hd)
    out = torch.empty(n, nh * hd, device=DEV, dtype=dtype)
    ops.attention_plain(to_dev(q), out, torch.tensor(positions, dtype=torch.int32, device=DEV),
                        torch.tensor(tok_seq, dtype=torch.int32, device=DEV), to_dev(tables), to_dev(ops.pack_keys(k_pages)),
                        to_dev(v_pages), nh, scale, window)
    want = plain_attention_rows(q, ks, vs, tok_seq, positions, nh, scale, window)
    tol = 2e-5 if dtype == torch.float32 else 2 ** -7
    err = (out.cpu().double() - want).abs().max().item()
    assert err < tol, err


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,nkv,hd,window,page", [(4, 2, 16, 0, 16), (8, 8, 64, 0, 16), (3, 1, 32, 0, 48), (8, 2, 128, 0, 32),
                                                   (2, 1, 256, 0, 64), (4, 2, 32, 300, 16), (5, 5, 80, 0, 64)])
def test_attention_plain_spread_over_workgroups_gives_the_bits_of_one_workgroup(dtype, nh, nkv, hd, window, page):
    """With a workspace the plain kernel gives every chunk of 256 keys a workgroup and merges them in a second kernel,
    by the same steps in the same order as one workgroup that walks them: bit for bit the same rows, and those of the
    float64 formula.  Contexts of one chunk, of a chunk and a key, of many; a window that starts inside a page."""
    from glassbox_amd import ops
    ctx_lens = [1, 256, 257, 1200, 700]
    k_pages, v_pages, tables, ks, vs = paged_setup(ctx_lens, nkv, hd, page, seed=hd + nh + page, dtype=dtype)
    tok_seq = [0, 1, 2, 3, 4, 3, 3]
    positions = [c - 1 for c in ctx_lens] + [600, 255]
    n = len(tok_seq)
    q = rnd(n, nh * hd, seed=12).to(dtype)
    scale = 1 / math.sqrt(hd)
    args = (torch.tensor(positions, dtype=torch.int32, device=DEV), torch.tensor(tok_seq, dtype=torch.int32, device=DEV),
            to_dev(tables), to_dev(ops.pack_keys(k_pages)), to_dev(v_pages), nh, scale, window)
    walked = torch.empty(n, nh * hd, device=DEV, dtype=dtype)
    ops.attention_plain(to_dev(q), walked, *args)
    floats = ops.attention_plain_split_floats(n, nh, hd, page, 1280)
    assert floats > 0
    ws = torch.full((floats,), float("nan"), device=DEV)
    spread = torch.empty(n, nh * hd, device=DEV, dtype=dtype)
    ops.attention_plain(to_dev(q), spread, *args, workspace=ws, max_context=1280)
    assert torch.equal(spread, walked)
    want = plain_attention_rows(q, ks, vs, tok_seq, positions, nh, scale, window)
    tol = 2e-5 if dtype == torch.float32 else 2 ** -7
    assert (walked.cpu().double() - want).abs().max().item() < tol
    # many (token, head) pairs, or contexts of one chunk: nothing to spread
    assert ops.attention_plain_split_floats(2000, nh, hd, page, 1280) == 0
    assert ops.attention_plain_split_floats(n, nh, hd, page, 256) == 0
    with pytest.raises(ops.KernelError, match="workspace"):
        ops.attention_plain(to_dev(q), spread, *args, workspace=ws[:100], max_context=1280)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,nkv,hd,page", [(4, 2, 16, 16), (8, 8, 64, 16), (3, 1, 32, 48), (2, 1, 128, 32), (2, 2, 256, 16),
                                            (5, 5, 80, 64)])
def test_attention_plain_eight_rows_a_workgroup_gives_the_bits_of_one_row_a_workgroup(dtype, nh, nkv, hd, page):
    """Many rows of prompt portions go eight rows a workgroup, which loads a key once where the eight are one request's
    consecutive tokens: bit for bit the rows of the one-row form.  Portions that start and end inside a group of
    eight, a group across the edge of a chunk of 256 keys (its first tokens have no key in the last chunk), single
    decoded tokens between portions; a head size and page for which the form is not built takes the one-row form."""
    from glassbox_amd import ops
    ctx_lens = [120, 263, 701, 531, 40]
    k_pages, v_pages, tables, ks, vs = paged_setup(ctx_lens, nkv, hd, page, seed=hd + nh + page + 1, dtype=dtype)
    rows = ([(0, p) for p in range(0, 101)]            # 101 rows: the next portion starts inside a group
            + [(1, p) for p in range(251, 262)]        # across key 256 in the middle of a group
            + [(2, 700)]                               # a decoded token
            + [(3, p) for p in range(509, 531)]        # across key 512
            + [(4, p) for p in range(0, 40)] + [(1, 262)])
    tok_seq, positions = [r[0] for r in rows], [r[1] for r in rows]
    n = len(rows)
    q = rnd(n, nh * hd, seed=14).to(dtype)
    scale = 1 / math.sqrt(hd)
    pos_d, seq_d = torch.tensor(positions, dtype=torch.int32, device=DEV), torch.tensor(tok_seq, dtype=torch.int32, device=DEV)
    rest = (to_dev(tables), to_dev(ops.pack_keys(k_pages)), to_dev(v_pages), nh, scale, 0)
    qd = to_dev(q)
    grouped = torch.empty(n, nh * hd, device=DEV, dtype=dtype)
    ops.attention_plain(qd, grouped, pos_d, seq_d, *rest, grouped=True)
    single = torch.empty(n, nh * hd, device=DEV, dtype=dtype)
    ops.attention_plain(qd, single, pos_d, seq_d, *rest)
    # the groups of eight fall elsewhere when the step's rows start at another row
    shifted = torch.empty(n, nh * hd, device=DEV, dtype=dtype)
    ops.attention_plain(qd[:3], shifted[:3], pos_d[:3], seq_d[:3], *rest, grouped=True)
    ops.attention_plain(qd[3:], shifted[3:], pos_d[3:], seq_d[3:], *rest, grouped=True)
    assert torch.equal(shifted, single)
    assert torch.equal(grouped, single)
    want = plain_attention_rows(q, ks, vs, tok_seq, positions, nh, scale, 0)
    tol = 2e-5 if dtype == torch.float32 else 2 ** -7
    assert (grouped.cpu().double() - want).abs().max().item() < tol


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_finds_one_far_key(dtype):
    """One key among hundreds is made to stand out: the output must be its value, wherever it lies
    (first or last slot of a page, first page, a page far away)."""
    from glassbox_amd import ops
    nh, nkv, hd, page, ctx = 4, 2, 32, 16, 700
    k_pages, v_pages, tables, ks, vs = paged_setup([ctx], nkv, hd, page, seed=1, dtype=dtype)
    q = rnd(1, nh * hd, seed=2).to(dtype)
    for target in (0, 15, 16, 255, 256, 511, 683, 699):
        kp = k_pages.clone()
        for kvh in range(nkv):
            # the key at `target` points along the mean query of its group, scaled up
            qg = q[0].float().reshape(nh, hd)[kvh * 2:(kvh + 1) * 2]
            key = torch.stack([qg[0], qg[1]]).mean(0)
            # make both heads of the group agree on the direction: use head 0's query for both
            kp[tables[0, target // page], kvh, target % page, :] = (qg[0] * 40).to(dtype)
        qq = q.clone().float().reshape(nh, hd)
        qq[1::2] = qq[0::2]   # both heads of a group ask the same
        qq = qq.reshape(1, nh * hd).to(dtype)
        out = torch.empty(1, nh * hd, device=DEV, dtype=dtype)
        ops.attention_plain(to_dev(qq), out, torch.tensor([ctx - 1], dtype=torch.int32, device=DEV),
                            torch.tensor([0], dtype=torch.int32, device=DEV), to_dev(tables), to_dev(ops.pack_keys(kp)),
                            to_dev(v_pages), nh, 1 / math.sqrt(hd), 0)
        want = vs[0][target].float().repeat_interleave(2, 0).reshape(-1)
        assert (out.cpu().float()[0] - want).abs().max().item() < 2e-2, f"key at {target} was not found"


class BareContext:
    """What the tuned attention bindings read from a step's context, for a hand-made batch: single-token
    requests first, then portions."""

    def __init__(self, q_lens, ctx_lens, tables, max_context=None):
        from types import SimpleNamespace
        self.num_seqs = len(q_lens)
        n_dec = sum(1 for l in q_lens if l == 1)
        assert all(l == 1 for l in q_lens[:n_dec]) and all(l > 1 for l in q_lens[n_dec:])
        q_start = np.concatenate([[0], np.cumsum(q_lens)[:-1]]).tolist()
        pos0 = [c - l for c, l in zip(ctx_lens, q_lens)]
        self.tok_seq = [s for s, l in enumerate(q_lens) for _ in range(l)]
        self.pos_list = [pos0[s] + j for s, l in enumerate(q_lens) for j in range(l)]
        i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
        self.positions, self.q_start, self.q_len, self.pos0 = i32(self.pos_list), i32(q_start), i32(q_lens), i32(pos0)
        self.tables = [to_dev(tables)]
        self.host = {"n_decode": n_dec, "max_q_len": max(q_lens), "max_context": max_context or max(ctx_lens)}
        self._bufs = {}

    def buffer(self, name, shape, dtype):
        return self._bufs.setdefault((name, tuple(shape)), torch.empty(shape, dtype=dtype, device=DEV))


@pytest.mark.parametrize("nh,nkv,hd,window", [(4, 2, 16, 0), (3, 1, 32, 0), (6, 2, 48, 0), (8, 8, 64, 0), (8, 2, 128, 0),
                                              (6, 3, 96, 0), (4, 4, 112, 0), (4, 2, 128, 70),
                                              (16, 1, 64, 0), (5, 5, 80, 0), (4, 2, 64, 37), (4, 4, 64, 300), (2, 1, 112, 0)])
@pytest.mark.parametrize("page", [16, 64])
def test_tuned_attention_against_the_plain_kernel(nh, nkv, hd, window, page):
    """The matrix-core kernels for decoding and for prompt portions against their plain twin and the
    float64 formula: contexts that end at every offset of a page, chunks that split, windows."""
    from types import SimpleNamespace
    from glassbox_amd import ops
    q_lens = [1, 1, 1, 1, 1, 5, 70, 16, 130]
    ctx_lens = [1, 17, 256, 700, 1025, 5, 300, 16, 530]      # portions 5/5, 70 ending at 300, 16/16, 130 ending at 530
    k_pages, v_pages, tables, ks, vs = paged_setup(ctx_lens, nkv, hd, page, seed=hd + nh, dtype=torch.bfloat16)
    ctx = BareContext(q_lens, ctx_lens, tables, max_context=1100)
    n = sum(q_lens)
    q = (rnd(n, nh * hd, seed=11) * 0.7).bfloat16()
    scale = 1 / math.sqrt(hd)
    cache = SimpleNamespace(k_pages=to_dev(ops.pack_keys(k_pages)), v_pages=to_dev(v_pages), group=0)
    assert ops.tuned_attention_supports(cache.k_pages, nh, window)
    out = torch.zeros(n, nh * hd, device=DEV, dtype=torch.bfloat16)
    qd = to_dev(q)
    ops.attention_decode(qd, out, ctx, cache, nh, scale, window)
    ops.attention_prefill(qd, out, ctx, cache, nh, scale, window)
    twin = torch.zeros_like(out)
    ops.attention_plain(qd, twin, ctx.positions, torch.tensor(ctx.tok_seq, dtype=torch.int32, device=DEV), ctx.tables[0],
                        cache.k_pages, cache.v_pages, nh, scale, window)
    want = plain_attention_rows(q, ks, vs, ctx.tok_seq, ctx.pos_list, nh, scale, window)
    err = (out.cpu().double() - want).abs().max(dim=1).values
    bad = torch.nonzero(err > 2 ** -6).flatten().tolist()
    assert not bad, f"rows {bad[:8]} (request, position) {[(ctx.tok_seq[i], ctx.pos_list[i]) for i in bad[:8]]}: {err[bad[:8]]}"
    # both are roundings to bfloat16 of nearly equal 32-bit results: at most a unit or two in the last place apart
    assert ((out.float() - twin.float()).abs() <= 2 ** -7 * (1 + twin.float().abs())).all()


@pytest.mark.parametrize("nh,nkv,hd,window", [(32, 32, 64, 0), (32, 8, 48, 0), (32, 4, 16, 100), (32, 32, 64, 200),
                                              (32, 16, 32, 0), (32, 8, 128, 0), (8, 8, 96, 0), (40, 8, 64, 0), (16, 4, 64, 0),
                                              (16, 16, 64, 150)])
def test_tuned_prefill_long_portions(nh, nkv, hd, window):
    """Portions long enough, and heads enough, that a wave takes 64 tokens: one portion starts in the
    middle of its request and ends off every tile edge, the other is a whole short prompt."""
    from types import SimpleNamespace
    from glassbox_amd import ops
    q_lens, ctx_lens = [1101, 300], [1303, 300]
    k_pages, v_pages, tables, ks, vs = paged_setup(ctx_lens, nkv, hd, 16, seed=hd + nh, dtype=torch.bfloat16)
    ctx = BareContext(q_lens, ctx_lens, tables)
    n = sum(q_lens)
    q = (rnd(n, nh * hd, seed=12) * 0.7).bfloat16()
    scale = 1 / math.sqrt(hd)
    cache = SimpleNamespace(k_pages=to_dev(ops.pack_keys(k_pages)), v_pages=to_dev(v_pages), group=0)
    out = torch.zeros(n, nh * hd, device=DEV, dtype=torch.bfloat16)
    qd = to_dev(q)
    ops.attention_prefill(qd, out, ctx, cache, nh, scale, window)
    twin = torch.zeros_like(out)
    ops.attention_plain(qd, twin, ctx.positions, torch.tensor(ctx.tok_seq, dtype=torch.int32, device=DEV), ctx.tables[0],
                        cache.k_pages, cache.v_pages, nh, scale, window)
    close = (out.float() - twin.float()).abs() <= 2 ** -7 * (1 + twin.float().abs())
    bad = torch.nonzero(~close.all(dim=1)).flatten().tolist()
    assert not bad, f"rows {bad[:8]} (request, position) {[(ctx.tok_seq[i], ctx.pos_list[i]) for i in bad[:8]]}"
    # a sample of rows against the formula in float64: tile edges, the portion's ends, the second request
    rows = [0, 1, 31, 32, 63, 64, 127, 128, 255, 256, 257, 700, 1023, 1024, 1099, 1100, 1101, 1102, 1400]
    want = plain_attention_rows(q[rows], ks, vs, [ctx.tok_seq[i] for i in rows], [ctx.pos_list[i] for i in rows], nh,
                                scale, window)
    err = (out[rows].cpu().double() - want).abs().max().item()
    assert err < 2 ** -6, err


@pytest.mark.parametrize("nh,nkv,hd,window", [(8, 8, 64, 0), (16, 8, 32, 0), (8, 8, 128, 0), (24, 8, 48, 200)])
def test_tuned_decode_with_a_workgroup_per_request_and_kv_head(nh, nkv, hd, window):
    """Requests and kv heads enough that no context is split over workgroups: sixteen waves share one,
    and their results are combined within the workgroup."""
    from types import SimpleNamespace
    from glassbox_amd import ops
    g = torch.Generator().manual_seed(nh + hd)
    ctx_lens = [1, 2, 63, 64, 65, 255, 256, 257, 1023, 1024, 1025, 1500] + torch.randint(1, 1400, (24,), generator=g).tolist()
    assert ops.decode_chunk(len(ctx_lens), nkv, 1536) >= 1536          # one chunk takes it all
    k_pages, v_pages, tables, ks, vs = paged_setup(ctx_lens, nkv, hd, 16, seed=hd, dtype=torch.bfloat16)
    ctx = BareContext([1] * len(ctx_lens), ctx_lens, tables, max_context=1536)
    n = len(ctx_lens)
    q = (rnd(n, nh * hd, seed=13) * 0.7).bfloat16()
    scale = 1 / math.sqrt(hd)
    cache = SimpleNamespace(k_pages=to_dev(ops.pack_keys(k_pages)), v_pages=to_dev(v_pages), group=0)
    out = torch.zeros(n, nh * hd, device=DEV, dtype=torch.bfloat16)
    ops.attention_decode(to_dev(q), out, ctx, cache, nh, scale, window)
    want = plain_attention_rows(q, ks, vs, ctx.tok_seq, ctx.pos_list, nh, scale, window)
    err = (out.cpu().double() - want).abs().max(dim=1).values
    bad = torch.nonzero(err > 2 ** -6).flatten().tolist()
    assert not bad, f"requests {bad[:8]} with contexts {[ctx_lens[i] for i in bad[:8]]}: {err[bad[:8]]}"


def test_tuned_decode_finds_one_far_key_in_every_chunk_position():
    """One key is made to stand out: first and last slot of a page, chunk edges, the last position."""
    from types import SimpleNamespace
    from glassbox_amd import ops
    nh, nkv, hd, page, ctxlen = 4, 2, 64, 16, 1500
    k_pages, v_pages, tables, ks, vs = paged_setup([ctxlen], nkv, hd, page, seed=1, dtype=torch.bfloat16)
    q = rnd(1, nh * hd, seed=2).float().reshape(nh, hd)
    q[1::2] = q[0::2]
    q = q.reshape(1, nh * hd).bfloat16()
    for target in (0, 15, 16, 63, 64, 255, 256, 257, 511, 512, 1023, 1024, 1279, 1280, 1498, 1499):
        kp = k_pages.clone()
        for kvh in range(nkv):
            kp[tables[0, target // page], kvh, target % page, :] = (q[0].float().reshape(nh, hd)[2 * kvh] * 40).bfloat16()
        for max_context in (1500, 4096):                       # one and several chunks per workgroup
            ctx = BareContext([1], [ctxlen], tables, max_context=max_context)
            out = torch.zeros(1, nh * hd, device=DEV, dtype=torch.bfloat16)
            cache = SimpleNamespace(k_pages=to_dev(ops.pack_keys(kp)), v_pages=to_dev(v_pages), group=0)
            ops.attention_decode(to_dev(q), out, ctx, cache, nh, 1 / math.sqrt(hd), 0)
            want = vs[0][target].float().repeat_interleave(2, 0).reshape(-1)
            assert (out.cpu().float()[0] - want).abs().max().item() < 2e-2, f"key at {target} was not found"


def test_tuned_decode_over_tens_of_thousands_of_keys():
    """Contexts of 40,000 and 33,333 keys beside one of 5: some hundred and sixty chunks a request for the second
    pass to merge, block tables of 2,500 pages.  Against the plain kernel on random keys, and with one key made to
    stand out near the start, in the middle and at the end."""
    from types import SimpleNamespace
    from glassbox_amd import ops
    nh, nkv, hd, page = 4, 2, 64, 16
    ctx_lens = [40000, 33333, 5]
    k_pages, v_pages, tables, ks, vs = paged_setup(ctx_lens, nkv, hd, page, seed=5, dtype=torch.bfloat16)
    q = (rnd(3, nh * hd, seed=6) * 0.7).bfloat16()
    ctx = BareContext([1, 1, 1], ctx_lens, tables, max_context=40960)
    assert -(-40960 // ops.decode_chunk(3, nkv, 40960)) > 100
    cache = SimpleNamespace(k_pages=to_dev(ops.pack_keys(k_pages)), v_pages=to_dev(v_pages), group=0)
    out, twin = (torch.zeros(3, nh * hd, device=DEV, dtype=torch.bfloat16) for _ in range(2))
    ops.attention_decode(to_dev(q), out, ctx, cache, nh, 1 / math.sqrt(hd), 0)
    ops.attention_plain(to_dev(q), twin, ctx.positions, torch.tensor([0, 1, 2], dtype=torch.int32, device=DEV), ctx.tables[0],
                        cache.k_pages, cache.v_pages, nh, 1 / math.sqrt(hd), 0)
    assert ((out.float() - twin.float()).abs() <= 2 ** -7 * (1 + twin.float().abs())).all()
    qq = q.float().reshape(3, nh, hd)
    qq[:, 1::2] = qq[:, 0::2]
    qq = qq.reshape(3, nh * hd).bfloat16()
    for target in (3, 20479, 20480, 39999):
        kp = k_pages.clone()
        for kvh in range(nkv):
            kp[tables[0, target // page], kvh, target % page, :] = (qq[0].float().reshape(nh, hd)[2 * kvh] * 40).bfloat16()
        cache = SimpleNamespace(k_pages=to_dev(ops.pack_keys(kp)), v_pages=to_dev(v_pages), group=0)
        ops.attention_decode(to_dev(qq), out, ctx, cache, nh, 1 / math.sqrt(hd), 0)
        want = vs[0][target].float().repeat_interleave(2, 0).reshape(-1)
        assert (out.cpu().float()[0] - want).abs().max().item() < 2e-2, f"key at {target} of 40,000 was not found"


@pytest.mark.parametrize("nh,nkv,hd,window", [(8, 2, 64, 0), (4, 4, 128, 0), (6, 3, 32, 700), (8, 8, 96, 0)])
def test_tuned_prefill_short_portions_over_long_contexts(nh, nkv, hd, window):
    """Few pairs of blocks and long contexts: several workgroups share a pair's keys and a second pass adds their
    sums.  Two short portions at the ends of long requests, beside a request of a single token."""
    from types import SimpleNamespace
    from glassbox_amd import ops
    q_lens, ctx_lens = [1, 100, 37], [400, 2150, 1301]
    k_pages, v_pages, tables, ks, vs = paged_setup(ctx_lens, nkv, hd, 16, seed=hd + nh, dtype=torch.bfloat16)
    ctx = BareContext(q_lens, ctx_lens, tables)
    lib = ops._lib("attention_bf16")
    assert lib.gb_attention_prefill_parts(max(q_lens), max(ctx_lens), nh, 2, hd) > 1
    n = sum(q_lens)
    q = (rnd(n, nh * hd, seed=14) * 0.7).bfloat16()
    scale = 1 / math.sqrt(hd)
    cache = SimpleNamespace(k_pages=to_dev(ops.pack_keys(k_pages)), v_pages=to_dev(v_pages), group=0)
    out = torch.zeros(n, nh * hd, device=DEV, dtype=torch.bfloat16)
    qd = to_dev(q)
    ops.attention_decode(qd, out, ctx, cache, nh, scale, window)
    ops.attention_prefill(qd, out, ctx, cache, nh, scale, window)
    twin = torch.zeros_like(out)
    ops.attention_plain(qd, twin, ctx.positions, torch.tensor(ctx.tok_seq, dtype=torch.int32, device=DEV), ctx.tables[0],
                        cache.k_pages, cache.v_pages, nh, scale, window)
    close = (out.float() - twin.float()).abs() <= 2 ** -7 * (1 + twin.float().abs())
    bad = torch.nonzero(~close.all(dim=1)).flatten().tolist()
    assert not bad, f"rows {bad[:8]} (request, position) {[(ctx.tok_seq[i], ctx.pos_list[i]) for i in bad[:8]]}"
    want = plain_attention_rows(q, ks, vs, ctx.tok_seq, ctx.pos_list, nh, scale, window)
    assert (out.cpu().double() - want).abs().max().item() < 2 ** -6
    again = torch.zeros_like(out)
    ops.attention_decode(qd, again, ctx, cache, nh, scale, window)
    ops.attention_prefill(qd, again, ctx, cache, nh, scale, window)
    assert torch.equal(out, again)


@pytest.mark.parametrize("nh,ctxlen,qlen", [(2, 200, 90), (64, 1200, 1090)])   # 32 and 64 tokens a wave
def test_tuned_prefill_sees_exactly_the_causal_keys(nh, ctxlen, qlen):
    """A portion in the middle of a request (it starts at position 110): token t must find a marked
    key at its own position and must not see the one after it."""
    from types import SimpleNamespace
    from glassbox_amd import ops
    nkv, hd, page = 2, 64, 16
    k_pages, v_pages, tables, ks, vs = paged_setup([ctxlen], nkv, hd, page, seed=3, dtype=torch.bfloat16)
    ctx = BareContext([qlen], [ctxlen], tables)
    # every key lies along one axis with a length that grows with its position, through consecutive
    # bfloat16 numbers from 16.0 on (so that rounding cannot reorder them): the newest visible key wins
    lengths = (torch.arange(ctxlen, dtype=torch.int32) + 0x4180).to(torch.int16).view(torch.bfloat16)
    axis = torch.zeros(hd)
    axis[5] = 1.0
    kp = k_pages.clone()
    for p in range(ctxlen):
        kp[tables[0, p // page], :, p % page, :] = (axis * lengths[p].float()).bfloat16()
    q = (axis * 768).repeat(qlen, nh).bfloat16()             # neighbours differ by 12 and more in score
    out = torch.zeros(qlen, nh * hd, device=DEV, dtype=torch.bfloat16)
    cache = SimpleNamespace(k_pages=to_dev(ops.pack_keys(kp)), v_pages=to_dev(v_pages), group=0)
    ops.attention_prefill(to_dev(q), out, ctx, cache, nh, 1 / math.sqrt(hd), 0)
    got = out.cpu().float().reshape(qlen, nkv, nh // nkv, hd)
    want = vs[0][110:110 + qlen].float()[:, :, None, :]      # not the value of the position after it
    worst = (got - want).abs().amax(dim=(1, 2, 3))
    assert worst.max().item() < 3e-2, f"token {int(worst.argmax())} of the portion"


def test_copy_rows():
    from glassbox_amd import ops
    base = rnd(6, 3, 10, seed=1).to(DEV)
    want = base.clone()
    want[4], want[0] = want[1].clone(), want[5].clone()
    ops.copy_rows(base, torch.tensor([1, 5], dtype=torch.int32, device=DEV), torch.tensor([4, 0], dtype=torch.int32, device=DEV))
    assert torch.equal(base, want)

