"""The benchmark configurations at their full sizes: each runs on the GPU exactly as bench.py runs it, and parts of the
result that the CPU checker can afford (whole images of a convolution, slabs of rows of a GEMM) are compared with the
oracle on the same operands; what is not sliceable (dedw's reduction over the whole batch) is tied to a sliceable
quantity by linearity."""
import numpy as np
import pytest

from intel_gaudi3_software_amd import ConvolutionParams, Epilogue, MmeSimTensor, abi
from helpers import A, bf16_bits_to_f32, decode_fp8, desc, quantize_fp8, rel_frobenius, to_bf16_bits

pytestmark = pytest.mark.gpu


def _dev(a):
    import torch
    return torch.from_numpy(a.view(np.int16) if a.dtype == np.uint16 else a).cuda()


def test_c2_fp8_gemm_full_size(calc, orc):
    """fp8_143 (bias 7) GEMM M = N = K = 4096 with per-tensor power-of-two scales and fused descale + bf16 output, exactly the
    benchmark's workload (same seed, operands quantised on the GPU by the cast kernel, which is bit-exact on its own): 16-row
    slabs out of four different row tiles (first and last rows of the matrix, and slabs that end at and straddle a 256-row
    tile boundary) plus 64 rows drawn at random, all 4096 columns each, against the oracle's accumulate -> descale -> cast."""
    import torch
    M = N = K = 4096
    rng = np.random.default_rng(2002)
    a32 = rng.standard_normal(M * K).astype(np.float32)
    b32 = rng.standard_normal(K * N).astype(np.float32)
    d_a32, d_b32 = torch.from_numpy(a32).cuda(), torch.from_numpy(b32).cuda()
    absmax = torch.zeros(2, dtype=torch.float32, device="cuda")
    calc.absmax(absmax[0:1], d_a32, M * K)
    calc.absmax(absmax[1:2], d_b32, K * N)
    calc.synchronize()
    assert float(absmax[0]) == float(np.abs(a32).max()) and float(absmax[1]) == float(np.abs(b32).max())
    eA, eB = (int(np.floor(np.log2(240.0 / float(v)))) for v in absmax.cpu())
    qa = torch.zeros(M * K, dtype=torch.uint8, device="cuda")
    qb = torch.zeros(K * N, dtype=torch.uint8, device="cuda")
    calc.castFromFp32(qa, abi.FP8_143, d_a32, M * K, fpBias=7, scale_exp=eA, clipFp=True)
    calc.castFromFp32(qb, abi.FP8_143, d_b32, K * N, fpBias=7, scale_exp=eB, clipFp=True)
    out = torch.zeros(M * N, dtype=torch.int16, device="cuda")
    X, Wt, Y = MmeSimTensor([K, M], 2, abi.FP8_143, qa, 7), MmeSimTensor([N, K], 2, abi.FP8_143, qb, 7), MmeSimTensor([N, M], 2, abi.BF16, out)
    calc.doBatchGemm(Y, X, Wt, abi.OP_AB, epilogue=Epilogue(scale_exp=-(eA + eB), clipFp=True))
    calc.synchronize()
    a8, b8 = qa.cpu().numpy().reshape(M, K), qb.cpu().numpy()
    got = out.cpu().numpy().view(np.uint16).reshape(M, N)
    rows = np.concatenate([np.arange(0, 16), np.arange(5 * 256 + 240, 5 * 256 + 256), np.arange(10 * 256 + 248, 10 * 256 + 264),
                           np.arange(M - 16, M), np.sort(np.random.default_rng(7).choice(M, 64, replace=False))])
    assert len({int(r) // 256 for r in rows}) >= 8  # the slabs alone cover tile rows 0, 5, 10, 11 and 15
    slab = np.ascontiguousarray(a8[rows].reshape(-1))
    acc = np.zeros(rows.size * N, np.float32)
    da, db, do = desc(slab, [K, rows.size], abi.FP8_143, 7), desc(b8, [N, K], abi.FP8_143, 7), desc(acc, [N, rows.size], abi.FP32)
    assert orc.orc_batch_gemm(A(do), A(da), A(db), abi.OP_AB) == 0
    want = np.zeros(rows.size * N, np.uint16)
    assert orc.orc_cast_from_fp32(want.ctypes.data, abi.BF16, 0, 0, acc.ctypes.data, rows.size * N, -(eA + eB), None, 0, 0, 0, 1, 0, 0) == 0
    g = got[rows].reshape(-1)
    dist = rel_frobenius(bf16_bits_to_f32(g), bf16_bits_to_f32(want))
    same = float(np.mean(g == want))
    print("c2 full size: %d rows, relative Frobenius distance of the bf16 outputs %.3e, %.2f %% of the codes equal" % (rows.size, dist, 100 * same))
    assert dist <= 1e-2  # the bound for fp8 operands
    assert dist <= 2e-3 and same >= 0.97  # what bf16 rounding of accumulators 1e-5 apart leaves
    assert np.count_nonzero(want & 0x7FFF) > want.size // 2
    # every row block of the output was written: no tile of the 16 x 16 grid is left at its initial zeros
    blocks = got.reshape(16, 256, 16, 256)
    assert np.all(np.count_nonzero(blocks & 0x7FFF, axis=(1, 3)) > 256 * 256 // 2)


def test_c3_conv_fwd_full_size(calc, orc):
    """bf16 3x3 forward convolution, N = 64, 56 x 56, 64 -> 64 channels, fused bf16 output: four whole images (first, last and
    two where a workgroup's run of rows starts in the middle of an image) against the oracle."""
    import torch
    rng = np.random.default_rng(1)
    B, H, W, Cc, Kk = 64, 56, 56, 64, 64
    xs, ws, ys = [Cc, W, H, 1, B], [Kk, Cc, 3, 3, 1], [Kk, W, H, 1, B]
    x = to_bf16_bits(np.maximum(rng.standard_normal(int(np.prod(xs))), 0).astype(np.float32))
    w = to_bf16_bits((rng.standard_normal(int(np.prod(ws))) * (2.0 / (Cc * 9)) ** 0.5).astype(np.float32))
    ty = torch.zeros(int(np.prod(ys)), dtype=torch.int16, device="cuda")
    cp = ConvolutionParams(2, [1, 1, 0, 0])
    X, Wt, Y = MmeSimTensor(xs, 5, abi.BF16, _dev(x)), MmeSimTensor(ws, 5, abi.BF16, _dev(w)), MmeSimTensor(ys, 5, abi.BF16, ty)
    calc.doConvolution(Y, X, Wt, Y, cp, abi.OP_FWD, epilogue=Epilogue(clipFp=True))
    calc.synchronize()
    got = ty.cpu().numpy().view(np.uint16).reshape(B, H * W * Kk)
    p = abi.make_conv_params(2, (1, 1, 0), (1, 1, 1), (1, 1, 1))
    per_img = H * W * Cc
    for b in (0, 17, 38, 63):
        xb = np.ascontiguousarray(x[b * per_img:(b + 1) * per_img])
        acc = np.zeros(H * W * Kk, np.float32)
        dx, dw, do = desc(xb, [Cc, W, H, 1, 1], abi.BF16), desc(w, ws, abi.BF16), desc(acc, [Kk, W, H, 1, 1], abi.FP32)
        assert orc.orc_convolution(A(do), A(dx), A(dw), A(do), A(p), abi.OP_FWD, 0) == 0
        want = bf16_bits_to_f32(to_bf16_bits(acc))
        g = bf16_bits_to_f32(got[b])
        assert rel_frobenius(g, want) <= 2e-3
        assert np.mean(got[b] == to_bf16_bits(acc)) >= 0.97


def test_c4_conv_dedx_dedw_full_size(calc, orc):
    """bf16 3x3 dedx / dedw, N = 32, 28 x 28, 256 -> 256 channels, fp32 outputs.  dedx: two whole images against the
    oracle.  dedw sums over the batch: the oracle's dedw of images 0 .. 1 must equal the GPU's full dedw minus the GPU's
    dedw of images 2 .. 31 (linearity in the batch)."""
    import torch
    rng = np.random.default_rng(2)
    B, H, W, Cc, Kk = 32, 28, 28, 256, 256
    xs, ws, ys = [Cc, W, H, 1, B], [Kk, Cc, 3, 3, 1], [Kk, W, H, 1, B]
    x = to_bf16_bits(np.maximum(rng.standard_normal(int(np.prod(xs))), 0).astype(np.float32))
    w = to_bf16_bits((rng.standard_normal(int(np.prod(ws))) * (2.0 / (Cc * 9)) ** 0.5).astype(np.float32))
    dy = to_bf16_bits((rng.standard_normal(int(np.prod(ys))) * 1e-2).astype(np.float32))
    cp = ConvolutionParams(2, [1, 1, 0, 0])
    p = abi.make_conv_params(2, (1, 1, 0), (1, 1, 1), (1, 1, 1))
    tx, tw, tdy = _dev(x), _dev(w), _dev(dy)
    X, Wt, DY = MmeSimTensor(xs, 5, abi.BF16, tx), MmeSimTensor(ws, 5, abi.BF16, tw), MmeSimTensor(ys, 5, abi.BF16, tdy)
    gdx = torch.zeros(int(np.prod(xs)), dtype=torch.float32, device="cuda")
    gdw = torch.zeros(int(np.prod(ws)), dtype=torch.float32, device="cuda")
    calc.doConvolution(MmeSimTensor(xs, 5, abi.FP32, gdx), X, Wt, DY, cp, abi.OP_DEDX)
    calc.doConvolution(MmeSimTensor(ws, 5, abi.FP32, gdw), X, Wt, DY, cp, abi.OP_DEDW)
    calc.synchronize()
    per_x, per_y = H * W * Cc, H * W * Kk
    dxg = gdx.cpu().numpy().reshape(B, per_x)
    for b in (0, 31):
        yb = np.ascontiguousarray(dy[b * per_y:(b + 1) * per_y])
        want = np.zeros(per_x, np.float32)
        ddy, dw, do = desc(yb, [Kk, W, H, 1, 1], abi.BF16), desc(w, ws, abi.BF16), desc(want, [Cc, W, H, 1, 1], abi.FP32)
        assert orc.orc_convolution(A(do), A(do), A(dw), A(ddy), A(p), abi.OP_DEDX, 0) == 0
        assert rel_frobenius(dxg[b], want) <= 2e-3
        assert rel_frobenius(dxg[b], want) <= 1e-4
    # dedw: oracle on the first two images; the GPU on the other thirty (views into the same device buffers)
    nb = 2
    want = np.zeros(int(np.prod(ws)), np.float32)
    x2, y2 = np.ascontiguousarray(x[:nb * per_x]), np.ascontiguousarray(dy[:nb * per_y])
    dx2, dy2, do = desc(x2, [Cc, W, H, 1, nb], abi.BF16), desc(y2, [Kk, W, H, 1, nb], abi.BF16), desc(want, ws, abi.FP32)
    assert orc.orc_convolution(A(do), A(dx2), A(do), A(dy2), A(p), abi.OP_DEDW, 0) == 0
    rest = torch.zeros(int(np.prod(ws)), dtype=torch.float32, device="cuda")
    Xr = MmeSimTensor([Cc, W, H, 1, B - nb], 5, abi.BF16, tx[nb * per_x:])
    Yr = MmeSimTensor([Kk, W, H, 1, B - nb], 5, abi.BF16, tdy[nb * per_y:])
    calc.doConvolution(MmeSimTensor(ws, 5, abi.FP32, rest), Xr, Wt, Yr, cp, abi.OP_DEDW)
    calc.synchronize()
    full, part = gdw.cpu().numpy().astype(np.float64), rest.cpu().numpy().astype(np.float64)
    # (the difference of two sums of 32 and 30 images carries their rounding: a few 1e-4 of the two-image result)
    assert rel_frobenius(full - part, want) <= 2e-3
    assert np.linalg.norm(want) > 0


def test_c5_batched_mixed_fp8_gemm_full_size(calc, orc):
    """Batched fp8 GEMM 4 x (2048 x 4096) x (4096 x 14336): A fp8_143 (bias 7), B fp8_152 (bias 15) shared by the batch,
    per-column power-of-two descale, fp8_143 output with saturation.  Slabs of 16 rows in all four batch elements against the
    oracle (accumulate, descale, cast): the first and the last tile row of the job, and tile rows in the middle of the walk
    over the tiles (batch elements 1 and 2, slabs that start inside a tile and one that straddles two tile rows).  Codes may
    differ by one where the accumulators straddle a rounding boundary."""
    import torch
    rng = np.random.default_rng(3)
    b5, M, K, N = 4, 2048, 4096, 14336
    a = rng.standard_normal((b5, M, K)).astype(np.float32)
    a[rng.random(a.shape) < 1e-3] *= 20.0
    sa = int(np.floor(np.log2(240.0 / np.abs(a).max())))
    qa = quantize_fp8(orc, a * np.float32(2.0 ** sa), abi.FP8_143, 7)
    wgt = (rng.standard_normal((K, N)) * 0.02).astype(np.float32)
    sb = np.floor(np.log2(57344.0 / np.abs(wgt).max(axis=0))).astype(np.int32)
    qb = quantize_fp8(orc, wgt * np.exp2(sb).astype(np.float32)[None, :], abi.FP8_152, 15)
    col = (-sb).astype(np.int32)
    out = torch.zeros(b5 * M * N, dtype=torch.uint8, device="cuda")
    A5 = MmeSimTensor([K, M, b5], 3, abi.FP8_143, _dev(qa.reshape(-1)), 7)
    B5 = MmeSimTensor([N, K, 1], 3, abi.FP8_152, _dev(qb.reshape(-1)), 15)
    Y5 = MmeSimTensor([N, M, b5], 3, abi.FP8_143, out, 7)
    # the product of the descales would leave tiny values: bring the result into the fp8_143 range with one more power of two
    extra = 6
    epi = Epilogue(scale_exp=-sa + extra, col_scale_exp=torch.from_numpy(col).cuda(), clipFp=True)
    calc.doBatchGemm(Y5, A5, B5, abi.OP_AB, epilogue=epi)
    calc.synchronize()
    got = out.cpu().numpy().reshape(b5, M, N)
    rows = 16
    for b, r0 in ((0, 0), (1, 3 * 256 + 40), (2, 5 * 256 - 8), (2, 1024 + 117), (3, M - rows)):
        slab = np.ascontiguousarray(qa[b, r0:r0 + rows].reshape(-1))
        acc = np.zeros(rows * N, np.float32)
        da, db, do = desc(slab, [K, rows], abi.FP8_143, 7), desc(qb.reshape(-1), [N, K], abi.FP8_152, 15), desc(acc, [N, rows], abi.FP32)
        assert orc.orc_batch_gemm(A(do), A(da), A(db), abi.OP_AB) == 0
        want = np.zeros(rows * N, np.uint8)
        assert orc.orc_cast_from_fp32(want.ctypes.data, abi.FP8_143, 7, 0, acc.ctypes.data, rows * N, -sa + extra, col.ctypes.data, N, 0, 0, 1, 0,
                                      0) == 0
        g = got[b, r0:r0 + rows].reshape(-1)
        assert np.mean(g == want) >= 0.97
        gf, wf = decode_fp8(orc, g, abi.FP8_143, 7), decode_fp8(orc, want, abi.FP8_143, 7)
        dist = rel_frobenius(gf, wf)
        print("c5 slab (batch %d, rows %d..): relative Frobenius distance of the fp8 outputs %.3e, %.2f %% of the codes equal" % (b, r0, dist, 100 * np.mean(g == want)))
        assert dist <= 1e-2
        assert np.count_nonzero(want & 0x7F) > rows * N // 2  # the slab is not a field of zeros


TILE_HEIGHT_TYPES = [(abi.BF16, abi.BF16, 0, 0), (abi.FP16, abi.FP16, 15, 15), (abi.FP8_143, abi.FP8_143, 7, 7), (abi.FP8_143, abi.FP8_152, 7, 15),
                     (abi.FP8_152, abi.FP8_143, 15, 11), (abi.FP8_152, abi.FP8_152, 20, 15)]


@pytest.mark.parametrize("dtA,dtB,bA,bB", TILE_HEIGHT_TYPES)
@pytest.mark.parametrize("op", [abi.OP_AB, abi.OP_ABT])
def test_large_tile_kernel_both_tile_heights(calc, orc, op, dtA, dtB, bA, bB):
    """The large-tile kernel picks 128-row tiles when 256-row tiles would occupy at most half of the compute units, else
    256-row ones.  A GEMM with 144 tiles of 256 x 256 (the 256-row kernel) and one with M = 384 (the 128-row kernel; M is
    not a multiple of 256), bf16, fp16 and every pair of fp8 flavours, both layouts of B: slabs of rows against the oracle."""
    import torch
    from helpers import random_operand
    rng = np.random.default_rng(3)
    for (M, N, K) in [(3072, 3072, 384), (384, 512, 512)]:
        a, b = random_operand(rng, dtA, M * K, orc, bA), random_operand(rng, dtB, N * K, orc, bB)
        bsz = [K, N] if op == abi.OP_ABT else [N, K]
        out = torch.zeros(M * N, dtype=torch.float32, device="cuda")
        calc.doBatchGemm(MmeSimTensor([N, M], 2, abi.FP32, out), MmeSimTensor([K, M], 2, dtA, _dev(a), bA), MmeSimTensor(bsz, 2, dtB, _dev(b), bB), op)
        calc.synchronize()
        got = out.cpu().numpy().reshape(M, N)
        for r0 in (0, M // 2 - 32, M - 64):
            slab = np.ascontiguousarray(a.reshape(M, K)[r0:r0 + 64])
            want = np.zeros(64 * N, np.float32)
            da, db, do = desc(slab, [K, 64], dtA, bA), desc(b, bsz, dtB, bB), desc(want, [N, 64], abi.FP32)
            assert orc.orc_batch_gemm(A(do), A(da), A(db), op) == 0
            assert rel_frobenius(got[r0:r0 + 64].ravel(), want) <= 1e-4, (M, r0)


@pytest.mark.parametrize("dt,dt_y,bias,bias_y", [(abi.BF16, abi.BF16, 0, 0), (abi.FP8_143, abi.FP8_152, 7, 15)])
def test_conv_gather_with_256_row_tiles(calc, orc, dt, dt_y, bias, bias_y):
    """A 3 x 3 forward convolution and dedx with enough pixels for more than 128 tiles of 256 rows (43 images of 28 x 28, 256
    channels: 132 tiles), so that the gather runs on the 256-row kernel (bf16, and fp8 with the gradient in the other fp8
    flavour); first and last image against the oracle."""
    import torch
    from helpers import random_operand
    rng = np.random.default_rng(4)
    B, H, W, Cc, Kk = 43, 28, 28, 256, 256
    xs, ws, ys = [Cc, W, H, 1, B], [Kk, Cc, 3, 3, 1], [Kk, W, H, 1, B]
    x = random_operand(rng, dt, int(np.prod(xs)), orc, bias)
    w = random_operand(rng, dt, int(np.prod(ws)), orc, bias, scale=0.05)
    dy = random_operand(rng, dt_y, int(np.prod(ys)), orc, bias_y)
    cp = ConvolutionParams(2, [1, 1, 0, 0])
    p = abi.make_conv_params(2, (1, 1, 0), (1, 1, 1), (1, 1, 1))
    X, Wt, DY = MmeSimTensor(xs, 5, dt, _dev(x), bias), MmeSimTensor(ws, 5, dt, _dev(w), bias), MmeSimTensor(ys, 5, dt_y, _dev(dy), bias_y)
    gy = torch.zeros(int(np.prod(ys)), dtype=torch.float32, device="cuda")
    gdx = torch.zeros(int(np.prod(xs)), dtype=torch.float32, device="cuda")
    out_y = MmeSimTensor(ys, 5, abi.FP32, gy)
    calc.doConvolution(out_y, X, Wt, out_y, cp, abi.OP_FWD)
    calc.doConvolution(MmeSimTensor(xs, 5, abi.FP32, gdx), X, Wt, DY, cp, abi.OP_DEDX)
    calc.synchronize()
    per_x, per_y = H * W * Cc, H * W * Kk
    yg, dxg = gy.cpu().numpy().reshape(B, per_y), gdx.cpu().numpy().reshape(B, per_x)
    for b in (0, B - 1):
        xb, yb = np.ascontiguousarray(x[b * per_x:(b + 1) * per_x]), np.ascontiguousarray(dy[b * per_y:(b + 1) * per_y])
        want_y, want_dx = np.zeros(per_y, np.float32), np.zeros(per_x, np.float32)
        dxb, dwd = desc(xb, [Cc, W, H, 1, 1], dt, bias), desc(w, ws, dt, bias)
        doy, dox, dyb = desc(want_y, [Kk, W, H, 1, 1], abi.FP32), desc(want_dx, [Cc, W, H, 1, 1], abi.FP32), desc(yb, [Kk, W, H, 1, 1], dt_y, bias_y)
        assert orc.orc_convolution(A(doy), A(dxb), A(dwd), A(doy), A(p), abi.OP_FWD, 0) == 0
        assert orc.orc_convolution(A(dox), A(dox), A(dwd), A(dyb), A(p), abi.OP_DEDX, 0) == 0
        assert rel_frobenius(yg[b], want_y) <= 1e-4 and rel_frobenius(dxg[b], want_dx) <= 1e-4
