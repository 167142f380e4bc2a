"""Convolution fwd / dedx / dedw on the GPU against the oracle (reference im2col + GEMM + col2im restated)."""
import numpy as np
import pytest

from intel_gaudi3_software_amd import ConvolutionParams, MmeSimTensor, abi
from helpers import A, TOL, desc, random_operand, rel_frobenius

pytestmark = pytest.mark.gpu


def _osz(i, k, p, s, d):
    return (i + 2 * p - d * (k - 1) - 1) // s + 1


# (C, K, W, H, D, B, S, R, Q, padding, stride, dilation, dim)
CASES = [
    (3, 4, 5, 5, 1, 2, 3, 3, 1, (1, 1, 0), (2, 2, 1), (1, 1, 1), 2),    # odd channels: element-wise loads
    (4, 3, 7, 6, 1, 2, 3, 2, 1, (2, 0, 0), (1, 2, 1), (2, 1, 1), 2),    # dilation, asymmetric padding
    (2, 3, 5, 4, 3, 1, 2, 2, 2, (1, 0, 1), (1, 1, 1), (1, 2, 1), 3),    # 3-d
    (16, 32, 9, 8, 1, 3, 3, 3, 1, (1, 1, 0), (1, 1, 1), (1, 1, 1), 2),  # vector loads
    (32, 16, 12, 10, 1, 2, 3, 3, 1, (1, 1, 0), (2, 2, 1), (1, 1, 1), 2),  # vector loads, stride 2 (dedx skips)
    (16, 16, 6, 6, 1, 1, 1, 1, 1, (0, 0, 0), (1, 1, 1), (1, 1, 1), 2),  # 1x1
]


def _run(calc, orc, case, dt, bias, op, device):
    import torch
    (C, K, W, H, D, B, S, R, Q, pad, st, dil, dim) = case
    rng = np.random.default_rng(100 + op)
    Wo, Ho, Do = _osz(W, S, pad[0], st[0], dil[0]), _osz(H, R, pad[1], st[1], dil[1]), _osz(D, Q, pad[2], st[2], dil[2])
    xs, ws, ys = [C, W, H, D, B], [K, C, S, R, Q], [K, Wo, Ho, Do, B]
    x = random_operand(rng, dt, int(np.prod(xs)), orc, bias)
    w = random_operand(rng, dt, int(np.prod(ws)), orc, bias, scale=0.3)
    y = random_operand(rng, dt, int(np.prod(ys)), orc, bias, scale=0.5)
    osz = {abi.OP_FWD: ys, abi.OP_DEDX: xs, abi.OP_DEDW: ws}[op]
    n = int(np.prod(osz))
    want = np.zeros(n, np.float32)
    p = abi.make_conv_params(dim, pad, st, dil)
    dx, dw, dy, do = desc(x, xs, dt, bias), desc(w, ws, dt, bias), desc(y, ys, dt, bias), desc(want, osz, abi.FP32)
    assert orc.orc_convolution(A(do), A(dx), A(dw), A(dy), A(p), op, 0) == 0, orc.orc_last_error()
    cp = ConvolutionParams(dim, list(pad) + [0], list(st) + [1], list(dil) + [1])
    if device:
        conv = (lambda a: torch.from_numpy(a.view(np.int16) if a.dtype.itemsize == 2 else a).cuda())
        tx, tw, ty = conv(x), conv(w), conv(y)
        to = torch.zeros(n, dtype=torch.float32, device="cuda")
        tens = {"x": MmeSimTensor(xs, 5, dt, tx, bias), "w": MmeSimTensor(ws, 5, dt, tw, bias), "y": MmeSimTensor(ys, 5, dt, ty, bias)}
        out = MmeSimTensor(osz, 5, abi.FP32, to)
        calc.doConvolution(out, tens["x"], tens["w"], tens["y"], cp, op)
        calc.synchronize()
        got = to.cpu().numpy()
    else:
        got = np.zeros(n, np.float32)
        calc.doConvolution(MmeSimTensor(osz, 5, abi.FP32, got), MmeSimTensor(xs, 5, dt, x, bias), MmeSimTensor(ws, 5, dt, w, bias),
                           MmeSimTensor(ys, 5, dt, y, bias), cp, op)
    return got, want


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("dt,bias", [(abi.BF16, 0), (abi.FP8_143, 7), (abi.FP32, 0)])
@pytest.mark.parametrize("op", [abi.OP_FWD, abi.OP_DEDX, abi.OP_DEDW])
def test_conv_vs_oracle(calc, orc, case, dt, bias, op):
    got, want = _run(calc, orc, case, dt, bias, op, device=(case[0] % 16 == 0))
    assert rel_frobenius(got, want) <= TOL[dt]
    # positions the reference leaves at exactly zero (dedx with stride > 1) must be exactly zero here as well
    assert np.all(got[want == 0] == 0) or op != abi.OP_DEDX


def _odd_strides(sizes, pads, order):
    """Element strides of a tensor whose dimensions 1 .. 4 lie in memory in the given order, each padded by pads[d] extra
    entries: rows that do not collapse to one pitch."""
    strides = [1, 0, 0, 0, 0]
    run = sizes[0] + pads[0]
    for d in order:
        strides[d] = run
        run *= sizes[d] + pads[d]
    return strides, run


@pytest.mark.parametrize("op", [abi.OP_FWD, abi.OP_DEDX, abi.OP_DEDW, abi.OP_TRANSPOSED_DEDX])
@pytest.mark.parametrize("dt,bias", [(abi.BF16, 0), (abi.FP8_152, 15)])
@pytest.mark.parametrize("device", [False, True])
def test_conv_tensors_with_arbitrary_strides(calc, orc, op, dt, bias, device):
    """Weights, activations, gradients and outputs whose dimensions are padded and stored in another order (rows without a
    common pitch): the reference follows any strides (createBufferWith/WithoutStrides, mme_reference_impl.cpp:245-319).
    Every logical element against the oracle reading the same buffers; what lies between the output's elements keeps its
    previous contents."""
    import torch
    rng = np.random.default_rng(300 + op)
    C, K, W, H, D, B, S, R, Q = 24, 40, 7, 6, 3, 2, 3, 2, 2
    pad, st, dil = (1, 0, 1), (1, 1, 1), (1, 1, 1)
    Wo, Ho, Do = _osz(W, S, pad[0], st[0], dil[0]), _osz(H, R, pad[1], st[1], dil[1]), _osz(D, Q, pad[2], st[2], dil[2])
    xs, ys = [C, W, H, D, B], [K, Wo, Ho, Do, B]
    ws = [C, K, S, R, Q] if op == abi.OP_TRANSPOSED_DEDX else [K, C, S, R, Q]
    (sx, nx), (sw, nw), (sy, ny) = _odd_strides(xs, [3, 1, 0, 2, 0], [2, 1, 4, 3]), _odd_strides(ws, [5, 2, 1, 0, 1], [3, 1, 2, 4]), \
        _odd_strides(ys, [1, 0, 2, 1, 1], [1, 3, 2, 4])
    x, w, y = random_operand(rng, dt, nx, orc, bias), random_operand(rng, dt, nw, orc, bias, scale=0.3), random_operand(rng, dt, ny, orc, bias, scale=0.5)
    osz, so, no = {abi.OP_FWD: (ys, sy, ny), abi.OP_DEDX: (xs, sx, nx), abi.OP_TRANSPOSED_DEDX: (xs, sx, nx), abi.OP_DEDW: (ws, sw, nw)}[op]
    want = np.full(no, 7.0, np.float32)
    p = abi.make_conv_params(3, pad, st, dil)
    dx, dw, dy, do = desc(x, xs, dt, bias, strides=sx), desc(w, ws, dt, bias, strides=sw), desc(y, ys, dt, bias, strides=sy), desc(want, osz, abi.FP32, strides=so)
    assert orc.orc_convolution(A(do), A(dx), A(dw), A(dy), A(p), op, 0) == 0, orc.orc_last_error()
    cp = ConvolutionParams(3, list(pad) + [0], list(st) + [1], list(dil) + [1])
    if device:
        conv = (lambda a: torch.from_numpy(a.view(np.int16) if a.dtype.itemsize == 2 else a).cuda())
        to = torch.full((no,), 7.0, dtype=torch.float32, device="cuda")
        calc.doConvolution(MmeSimTensor(osz, 5, abi.FP32, to, strides=so), MmeSimTensor(xs, 5, dt, conv(x), bias, strides=sx),
                           MmeSimTensor(ws, 5, dt, conv(w), bias, strides=sw), MmeSimTensor(ys, 5, dt, conv(y), bias, strides=sy), cp, op)
        calc.synchronize()
        got = to.cpu().numpy()
    else:
        got = np.full(no, 7.0, np.float32)
        calc.doConvolution(MmeSimTensor(osz, 5, abi.FP32, got, strides=so), MmeSimTensor(xs, 5, dt, x, bias, strides=sx),
                           MmeSimTensor(ws, 5, dt, w, bias, strides=sw), MmeSimTensor(ys, 5, dt, y, bias, strides=sy), cp, op)
    # the tensor's own elements
    idx = np.zeros(osz[::-1], np.int64)
    for d, (n, stv) in enumerate(zip(osz, so)):
        shape = [1] * 5
        shape[4 - d] = n
        idx = idx + (np.arange(n, dtype=np.int64) * stv).reshape(shape)
    idx = idx.ravel()
    assert rel_frobenius(got[idx], want[idx]) <= TOL[dt] and np.any(want[idx] != 7.0)
    rest = np.ones(no, bool)
    rest[idx] = False
    assert np.all(got[rest] == 7.0)


def test_conv_fwd_bounded_waits_report_instead_of_hanging(orc):
    """The 3 x 3 forward kernels hand rows between wavefronts through counters in LDS and poll them a bounded number of
    times.  With the bound forced to zero from the host a wavefront that has to wait at all gives up at once: the kernel
    still ends normally and the next synchronize() reports it; with the bound restored the same call is right again.  Both
    forms of the kernel: the one that keeps a workgroup's rows resident in LDS and the two-team one."""
    import torch
    from intel_gaudi3_software_amd import HipCalculator
    from intel_gaudi3_software_amd.calculator import MMEStackException
    from helpers import bf16_bits_to_f32, to_bf16_bits
    rng = np.random.default_rng(55)
    calc = HipCalculator()
    gave_up = []
    try:
        for B, H, W in [(8, 56, 56), (256, 56, 56)]:
            Cc = Kk = 64
            xs, ws, ys = [Cc, W, H, 1, B], [Kk, Cc, 3, 3, 1], [Kk, W, H, 1, B]
            x = to_bf16_bits(np.maximum(rng.standard_normal(int(np.prod(xs))), 0).astype(np.float32))
            w = to_bf16_bits((rng.standard_normal(int(np.prod(ws))) * 0.06).astype(np.float32))
            tx, tw = torch.from_numpy(x.view(np.int16)).cuda(), torch.from_numpy(w.view(np.int16)).cuda()
            ty = torch.zeros(int(np.prod(ys)), dtype=torch.float32, device="cuda")
            X, Wt, Y = MmeSimTensor(xs, 5, abi.BF16, tx), MmeSimTensor(ws, 5, abi.BF16, tw), MmeSimTensor(ys, 5, abi.FP32, ty)
            cp = ConvolutionParams(2, [1, 1, 0, 0])
            calc.setWaitLimit(0)
            print("bounded waits: limit 0,", B, H, W, flush=True)
            calc.doConvolution(Y, X, Wt, Y, cp, abi.OP_FWD)
            try:
                calc.synchronize()
                gave_up.append(False)
            except MMEStackException as e:
                assert "bounded wait" in str(e) and e.status == abi.EHIP
                gave_up.append(True)
            calc.setWaitLimit(1 << 22)
            print("bounded waits: limit restored,", B, H, W, flush=True)
            calc.doConvolution(Y, X, Wt, Y, cp, abi.OP_FWD)
            calc.synchronize()   # no report this time
            got = ty.cpu().numpy().reshape(B, H * W * Kk)
            b = B - 1
            xb = np.ascontiguousarray(x[b * H * W * Cc:(b + 1) * H * W * Cc])
            want = np.zeros(H * W * Kk, np.float32)
            p = abi.make_conv_params(2, (1, 1, 0), (1, 1, 1), (1, 1, 1))
            dx, dw, do = desc(xb, [Cc, W, H, 1, 1], abi.BF16), desc(w, ws, abi.BF16), desc(want, [Kk, W, H, 1, 1], abi.FP32)
            assert orc.orc_convolution(A(do), A(dx), A(dw), A(do), A(p), abi.OP_FWD, 0) == 0
            assert rel_frobenius(got[b], want) <= 1e-4
    finally:
        calc.close()
    assert any(gave_up), "no wavefront ever had to wait: the report path was not exercised"


def test_conv_adjoint_identities(calc, orc):
    """<dY, fwd(X, W)> = <dedx(dY, W), X> = <dedw(X, dY), W> on a shape too large for the oracle to do quickly."""
    import torch
    rng = np.random.default_rng(77)
    C, K, W, H, B = 64, 64, 28, 28, 8
    xs, ws, ys = [C, W, H, 1, B], [K, C, 3, 3, 1], [K, W, H, 1, B]
    from helpers import bf16_bits_to_f32, to_bf16_bits
    x = to_bf16_bits(rng.standard_normal(int(np.prod(xs))))
    w = to_bf16_bits(rng.standard_normal(int(np.prod(ws))) * 0.1)
    dy = to_bf16_bits(rng.standard_normal(int(np.prod(ys))))
    conv = lambda a: torch.from_numpy(a.view(np.int16)).cuda()
    tx, tw, ty = conv(x), conv(w), conv(dy)
    X, Wt, Y = MmeSimTensor(xs, 5, abi.BF16, tx), MmeSimTensor(ws, 5, abi.BF16, tw), MmeSimTensor(ys, 5, abi.BF16, ty)
    cp = ConvolutionParams(2, [1, 1, 0, 0], [1, 1, 1, 1], [1, 1, 1, 1])
    f = torch.zeros(int(np.prod(ys)), dtype=torch.float32, device="cuda")
    gx = torch.zeros(int(np.prod(xs)), dtype=torch.float32, device="cuda")
    gw = torch.zeros(int(np.prod(ws)), dtype=torch.float32, device="cuda")
    calc.doConvolution(MmeSimTensor(ys, 5, abi.FP32, f), X, Wt, Y, cp, abi.OP_FWD)
    calc.doConvolution(MmeSimTensor(xs, 5, abi.FP32, gx), X, Wt, Y, cp, abi.OP_DEDX)
    calc.doConvolution(MmeSimTensor(ws, 5, abi.FP32, gw), X, Wt, Y, cp, abi.OP_DEDW)
    calc.synchronize()
    xf, wf, yf = (bf16_bits_to_f32(v).astype(np.float64) for v in (x, w, dy))
    s_f = np.dot(yf, f.cpu().numpy().astype(np.float64))
    s_x = np.dot(xf, gx.cpu().numpy().astype(np.float64))
    s_w = np.dot(wf, gw.cpu().numpy().astype(np.float64))
    assert abs(s_f - s_x) <= 1e-4 * abs(s_f) and abs(s_f - s_w) <= 1e-4 * abs(s_f)


@pytest.mark.parametrize("B,H,W", [(2, 11, 13), (1, 8, 56), (3, 17, 7)])
def test_conv_fwd_fast_path_vs_oracle(calc, orc, B, H, W):
    """The specialised forward kernel (bf16, 3x3, 64 -> 64, stride 1, padding 1): ragged heights / widths, fp32
    accumulators against the oracle and the fused bf16 output against the oracle cast of the same accumulators."""
    import torch
    from intel_gaudi3_software_amd import Epilogue
    from helpers import to_bf16_bits
    rng = np.random.default_rng(500 + H)
    xs, ws, ys = [64, W, H, 1, B], [64, 64, 3, 3, 1], [64, W, H, 1, B]
    x = to_bf16_bits(np.maximum(rng.standard_normal(int(np.prod(xs))), 0))
    w = to_bf16_bits(rng.standard_normal(int(np.prod(ws))) * (2.0 / 576) ** 0.5)
    want = np.zeros(int(np.prod(ys)), np.float32)
    p = abi.make_conv_params(2, (1, 1, 0), (1, 1, 1), (1, 1, 1))
    dx, dw, dy = desc(x, xs, abi.BF16), desc(w, ws, abi.BF16), desc(want, ys, abi.FP32)
    assert orc.orc_convolution(A(dy), A(dx), A(dw), A(dy), A(p), abi.OP_FWD, 0) == 0
    tx, tw = torch.from_numpy(x.view(np.int16)).cuda(), torch.from_numpy(w.view(np.int16)).cuda()
    acc = torch.zeros(want.size, dtype=torch.float32, device="cuda")
    out = torch.zeros(want.size, dtype=torch.int16, device="cuda")
    X, Wt = MmeSimTensor(xs, 5, abi.BF16, tx), MmeSimTensor(ws, 5, abi.BF16, tw)
    cp = ConvolutionParams(2, [1, 1, 0, 0], [1, 1, 1, 1], [1, 1, 1, 1])
    calc.doConvolution(MmeSimTensor(ys, 5, abi.FP32, acc), X, Wt, MmeSimTensor(ys, 5, abi.FP32, acc), cp, abi.OP_FWD)
    calc.doConvolution(MmeSimTensor(ys, 5, abi.BF16, out), X, Wt, MmeSimTensor(ys, 5, abi.BF16, out), cp, abi.OP_FWD,
                       epilogue=Epilogue(scale_exp=1, relu=True, clipFp=True))
    calc.synchronize()
    got = acc.cpu().numpy()
    assert rel_frobenius(got, want) <= 2e-3
    assert rel_frobenius(got, want) <= 1e-4
    want16 = np.zeros(want.size, np.uint16)
    assert orc.orc_cast_from_fp32(want16.ctypes.data, abi.BF16, 0, 0, got.ctypes.data, got.size, 1, None, 0, 1, 0, 1, 0, 0) == 0
    assert np.array_equal(out.cpu().numpy().view(np.uint16), want16)


@pytest.mark.parametrize("relu,clip", [(False, False), (True, False), (False, True), (True, True)])
def test_conv_fwd_fast_path_special_values(calc, orc, relu, clip):
    """inf, NaN and huge activations through the specialised forward kernel with an unscaled bf16 epilogue: the
    blocks that hold NaN / inf / overflow leave the hardware-convert path for the exact converter; bit-exact against the
    oracle cast (relu, clipping) of the kernel's own fp32 accumulators."""
    import torch
    from intel_gaudi3_software_amd import Epilogue
    from helpers import to_bf16_bits
    rng = np.random.default_rng(900)
    B, H, W = 2, 9, 21
    xs, ws, ys = [64, W, H, 1, B], [64, 64, 3, 3, 1], [64, W, H, 1, B]
    x = to_bf16_bits(rng.standard_normal(int(np.prod(xs))))
    w = to_bf16_bits(rng.standard_normal(int(np.prod(ws))) * 0.05)
    xv = x.reshape(B, H, W, 64)
    xv[0, 2, 3, 5] = 0x7F80   # +inf
    xv[0, 6, 17, 9] = 0xFF80  # -inf
    xv[1, 4, 4, 0] = 0x7FC0   # NaN
    xv[1, 7, 12, :] = 0x7F00  # 1.7e38 in every channel: sums overflow bf16 and fp32
    tx, tw = torch.from_numpy(x.view(np.int16)).cuda(), torch.from_numpy(w.view(np.int16)).cuda()
    n = int(np.prod(ys))
    acc = torch.zeros(n, dtype=torch.float32, device="cuda")
    out = torch.zeros(n, dtype=torch.int16, device="cuda")
    X, Wt = MmeSimTensor(xs, 5, abi.BF16, tx), MmeSimTensor(ws, 5, abi.BF16, tw)
    cp = ConvolutionParams(2, [1, 1, 0, 0], [1, 1, 1, 1], [1, 1, 1, 1])
    calc.doConvolution(MmeSimTensor(ys, 5, abi.FP32, acc), X, Wt, MmeSimTensor(ys, 5, abi.FP32, acc), cp, abi.OP_FWD)
    calc.doConvolution(MmeSimTensor(ys, 5, abi.BF16, out), X, Wt, MmeSimTensor(ys, 5, abi.BF16, out), cp, abi.OP_FWD,
                       epilogue=Epilogue(relu=relu, clipFp=clip))
    calc.synchronize()
    got = acc.cpu().numpy()
    assert np.isnan(got).any() and np.isinf(got).any()
    want16 = np.zeros(n, np.uint16)
    assert orc.orc_cast_from_fp32(want16.ctypes.data, abi.BF16, 0, 0, got.ctypes.data, n, 0, None, 0, int(relu), 0, int(clip), 0, 0) == 0
    assert np.array_equal(out.cpu().numpy().view(np.uint16), want16)


# shapes that take the large-tile kernel with the gather on its load side: 2-byte operands, at least 128 output columns (a
# multiple of 16: the last column tile may be partial), channel counts that are multiples of 32; ragged pixel counts,
# dilation, a strided forward pass, a 1 x 1 filter
GATHER_CASES = [
    (256, 256, 9, 7, 1, 2, 3, 3, 1, (1, 1, 0), (1, 1, 1), (1, 1, 1), 2),
    (64, 256, 11, 6, 1, 1, 3, 3, 1, (2, 2, 0), (1, 1, 1), (2, 2, 1), 2),
    (256, 256, 8, 8, 1, 1, 1, 1, 1, (0, 0, 0), (1, 1, 1), (1, 1, 1), 2),
    (128, 192, 10, 7, 1, 2, 3, 3, 1, (1, 1, 0), (1, 1, 1), (1, 1, 1), 2),   # fwd: 192 columns, dedx: 128 (partial column tiles)
    (160, 400, 6, 5, 1, 3, 3, 3, 1, (1, 1, 0), (1, 1, 1), (1, 1, 1), 2),    # fwd: two column tiles, the second partial
]


# the gather's padding lanes read a page of zeros as long as a tap's channels may be (4096 bytes): 2048 bf16 channels still
# take the large-tile kernel (every lane of a padded tap walks to the page's last 64 bytes), 2112 are routed to the general
# kernel; the gathered tensor is x for fwd (C channels) and dy for dedx (K channels)
@pytest.mark.parametrize("op,C,K", [(abi.OP_FWD, 2048, 128), (abi.OP_FWD, 2112, 128), (abi.OP_DEDX, 128, 2048), (abi.OP_DEDX, 128, 2112)])
def test_conv_gather_with_as_many_channels_as_the_zero_page_holds(calc, orc, op, C, K):
    case = (C, K, 6, 5, 1, 1, 3, 3, 1, (1, 1, 0), (1, 1, 1), (1, 1, 1), 2)
    got, want = _run(calc, orc, case, abi.BF16, 0, op, device=True)
    assert rel_frobenius(got, want) <= 1e-4


@pytest.mark.parametrize("case", GATHER_CASES)
@pytest.mark.parametrize("op", [abi.OP_FWD, abi.OP_DEDX])
@pytest.mark.parametrize("dt,bias", [(abi.BF16, 0), (abi.FP16, 15), (abi.FP16, 11), (abi.FP8_143, 7), (abi.FP8_143, 11), (abi.FP8_152, 15)])
def test_conv_large_tile_gather_vs_oracle(calc, orc, case, op, dt, bias):
    # (dedx has C output columns and the large-tile kernel takes 128 or more: the dedx of the 64-channel case runs on the
    # general kernel, and is held to the same bounds)
    got, want = _run(calc, orc, case, dt, bias, op, device=True)
    assert rel_frobenius(got, want) <= TOL[dt]
    assert rel_frobenius(got, want) <= 1e-4


# dedw on the large-tile kernel: pixels (the reduction) a multiple of 64 and at least 192, K a multiple of 256 output columns.
# Up to 128 tiles of 256 x 256 the kernel runs with 128-row tiles (the first three cases), beyond that with 256-row ones
# (the last case: 9 x 15 tiles).
DEDW_CASES = [
    (256, 256, 8, 8, 1, 3, 3, 3, 1, (1, 1, 0), (1, 1, 1), (1, 1, 1), 2),
    (64, 256, 16, 8, 1, 2, 3, 3, 1, (2, 2, 0), (1, 1, 1), (2, 2, 1), 2),     # M = 576: ragged row tile, three taps per tile
    (32, 256, 18, 17, 1, 1, 3, 3, 1, (0, 0, 0), (2, 2, 1), (1, 1, 1), 2),    # strided: 8 x 8 output pixels
    (256, 3840, 8, 8, 1, 3, 3, 3, 1, (1, 1, 0), (1, 1, 1), (1, 1, 1), 2),
    (96, 208, 16, 12, 1, 1, 3, 3, 1, (1, 1, 0), (1, 1, 1), (1, 1, 1), 2),      # 208 output columns: a partial column tile
    (64, 256, 16, 8, 1, 3, 3, 3, 1, (1, 1, 0), (1, 1, 1), (1, 1, 1), 2),       # 384 pixels: enough for the fp8 kernel's k-stages
]


@pytest.mark.parametrize("case", DEDW_CASES)
@pytest.mark.parametrize("dt,bias", [(abi.BF16, 0), (abi.FP16, 15), (abi.FP8_143, 7), (abi.FP8_152, 15)])
def test_conv_large_tile_dedw_vs_oracle(calc, orc, case, dt, bias):
    got, want = _run(calc, orc, case, dt, bias, abi.OP_DEDW, device=True)
    assert rel_frobenius(got, want) <= TOL[dt]
    assert rel_frobenius(got, want) <= 1e-4


def test_conv_large_tile_strided_forward_vs_oracle(calc, orc):
    case = (64, 256, 13, 9, 1, 2, 3, 3, 1, (1, 1, 0), (2, 2, 1), (1, 1, 1), 2)
    got, want = _run(calc, orc, case, abi.BF16, 0, abi.OP_FWD, device=True)
    assert rel_frobenius(got, want) <= 1e-4


def test_conv_adjoint_identities_256_channels(calc, orc):
    """<dY, fwd(X, W)> = <dedx(dY, W), X> = <dedw(X, dY), W> with 256 channels: fwd and dedx on the large-tile kernel (four
    tiles, the last one ragged), dedw on the general kernel."""
    import torch
    rng = np.random.default_rng(78)
    C, K, W, H, B = 256, 256, 14, 14, 4
    xs, ws, ys = [C, W, H, 1, B], [K, C, 3, 3, 1], [K, W, H, 1, B]
    from helpers import bf16_bits_to_f32, to_bf16_bits
    x = to_bf16_bits(rng.standard_normal(int(np.prod(xs))))
    w = to_bf16_bits(rng.standard_normal(int(np.prod(ws))) * 0.05)
    dy = to_bf16_bits(rng.standard_normal(int(np.prod(ys))))
    conv = lambda a: torch.from_numpy(a.view(np.int16)).cuda()
    tx, tw, ty = conv(x), conv(w), conv(dy)
    X, Wt, Y = MmeSimTensor(xs, 5, abi.BF16, tx), MmeSimTensor(ws, 5, abi.BF16, tw), MmeSimTensor(ys, 5, abi.BF16, ty)
    cp = ConvolutionParams(2, [1, 1, 0, 0], [1, 1, 1, 1], [1, 1, 1, 1])
    f = torch.zeros(int(np.prod(ys)), dtype=torch.float32, device="cuda")
    gx = torch.zeros(int(np.prod(xs)), dtype=torch.float32, device="cuda")
    gw = torch.zeros(int(np.prod(ws)), dtype=torch.float32, device="cuda")
    calc.doConvolution(MmeSimTensor(ys, 5, abi.FP32, f), X, Wt, Y, cp, abi.OP_FWD)
    calc.doConvolution(MmeSimTensor(xs, 5, abi.FP32, gx), X, Wt, Y, cp, abi.OP_DEDX)
    calc.doConvolution(MmeSimTensor(ws, 5, abi.FP32, gw), X, Wt, Y, cp, abi.OP_DEDW)
    calc.synchronize()
    xf, wf, yf = (bf16_bits_to_f32(v).astype(np.float64) for v in (x, w, dy))
    s_f = np.dot(yf, f.cpu().numpy().astype(np.float64))
    s_x = np.dot(xf, gx.cpu().numpy().astype(np.float64))
    s_w = np.dot(wf, gw.cpu().numpy().astype(np.float64))
    assert abs(s_f - s_x) <= 1e-4 * abs(s_f) and abs(s_f - s_w) <= 1e-4 * abs(s_f)


@pytest.mark.parametrize("dt,bias", [(abi.BF16, 0), (abi.FP8_143, 7), (abi.FP32, 0)])
@pytest.mark.parametrize("case", [CASES[0], CASES[1], (64, 128, 9, 8, 1, 4, 3, 3, 1, (1, 1, 0), (1, 1, 1), (1, 1, 1), 2)])
def test_transposed_dedx(calc, orc, case, dt, bias):
    """transposed_dedx takes the weights with their first two dimensions exchanged and reads them with the S axis
    reversed (mme_reference_impl.cpp:625-647).  Against the oracle (which is pinned against the compiled reference for
    this op), and bit for bit against the library's own dedx on explicitly transposed and reversed weights."""
    import torch
    (C, K, W, H, D, B, S, R, Q, pad, st, dil, dim) = case
    rng = np.random.default_rng(300)
    Wo, Ho, Do = _osz(W, S, pad[0], st[0], dil[0]), _osz(H, R, pad[1], st[1], dil[1]), _osz(D, Q, pad[2], st[2], dil[2])
    xs, wts, ys = [C, W, H, D, B], [C, K, S, R, Q], [K, Wo, Ho, Do, B]
    wt = random_operand(rng, dt, int(np.prod(wts)), orc, bias, scale=0.3)
    y = random_operand(rng, dt, int(np.prod(ys)), orc, bias, scale=0.5)
    n = int(np.prod(xs))
    want = np.zeros(n, np.float32)
    p = abi.make_conv_params(dim, pad, st, dil)
    dw, dy, do = desc(wt, wts, dt, bias), desc(y, ys, dt, bias), desc(want, xs, abi.FP32)
    assert orc.orc_convolution(A(do), A(do), A(dw), A(dy), A(p), abi.OP_TRANSPOSED_DEDX, 0) == 0, orc.orc_last_error()
    cp = ConvolutionParams(dim, list(pad) + [0], list(st) + [1], list(dil) + [1])
    conv = (lambda a: torch.from_numpy(a.view(np.int16) if dt == abi.BF16 else a).cuda())
    tw, ty = conv(wt), conv(y)
    got = torch.zeros(n, dtype=torch.float32, device="cuda")
    X = MmeSimTensor(xs, 5, abi.FP32, got)
    calc.doConvolution(X, X, MmeSimTensor(wts, 5, dt, tw, bias), MmeSimTensor(ys, 5, dt, ty, bias), cp, abi.OP_TRANSPOSED_DEDX)
    # the same through plain dedx: w[k][c][s][r][q] = wt[c][k][S - 1 - s][r][q]
    w5 = wt.reshape(Q, R, S, K, C)  # numpy order: last index = contiguous dimension (c)
    w_plain = np.ascontiguousarray(w5[:, :, ::-1, :, :].transpose(0, 1, 2, 4, 3)).reshape(-1)
    got2 = torch.zeros(n, dtype=torch.float32, device="cuda")
    X2 = MmeSimTensor(xs, 5, abi.FP32, got2)
    calc.doConvolution(X2, X2, MmeSimTensor([K, C, S, R, Q], 5, dt, conv(w_plain), bias), MmeSimTensor(ys, 5, dt, ty, bias), cp, abi.OP_DEDX)
    calc.synchronize()
    g1, g2 = got.cpu().numpy(), got2.cpu().numpy()
    assert np.array_equal(g1.view(np.uint32), g2.view(np.uint32))
    assert rel_frobenius(g1, want) <= (1e-2 if dt == abi.FP8_143 else 2e-3)


@pytest.mark.parametrize("op", [abi.OP_FWD, abi.OP_DEDX, abi.OP_DEDW])
@pytest.mark.parametrize("pitch_extra", [1, 8])
def test_conv_weights_with_a_row_pitch(calc, orc, op, pitch_extra):
    """Weight tensors whose rows of K output channels are spaced wider than K (the reference's strided-tensor tests give w such
    strides): read by fwd and dedx, written by dedw, whose gap columns must keep their contents."""
    C, K, W, H, B, S, R = 16, 24, 9, 8, 2, 3, 3
    rng = np.random.default_rng(300 + op)
    xs, ws, ys = [C, W, H, 1, B], [K, C, S, R, 1], [K, W, H, 1, B]
    ld = K + pitch_extra
    wstr = [1, ld, ld * C, ld * C * S, ld * C * S * R]
    x = random_operand(rng, abi.BF16, int(np.prod(xs)))
    y = random_operand(rng, abi.BF16, int(np.prod(ys)), scale=0.5)
    w = random_operand(rng, abi.BF16, ld * C * S * R, scale=0.3)
    p = abi.make_conv_params(2, (1, 1, 0), (1, 1, 1), (1, 1, 1))
    cp = ConvolutionParams(2, [1, 1, 0, 0], [1, 1, 1, 1], [1, 1, 1, 1])
    if op == abi.OP_DEDW:
        want = np.full(ld * C * S * R, 7.0, np.float32)
        got = want.copy()
        do = desc(want, ws, abi.FP32, strides=wstr)
        dx, dy = desc(x, xs, abi.BF16), desc(y, ys, abi.BF16)
        assert orc.orc_convolution(A(do), A(dx), A(do), A(dy), A(p), op, 0) == 0, orc.orc_last_error()
        out = MmeSimTensor(ws, 5, abi.FP32, got, strides=wstr)
        calc.doConvolution(out, MmeSimTensor(xs, 5, abi.BF16, x), out, MmeSimTensor(ys, 5, abi.BF16, y), cp, op)
        gaps = np.ones(want.size, bool).reshape(-1, ld)
        gaps[:, :K] = False
        assert np.all(got.reshape(-1, ld)[gaps] == 7.0)
    else:
        osz = ys if op == abi.OP_FWD else xs
        want, got = np.zeros(int(np.prod(osz)), np.float32), np.zeros(int(np.prod(osz)), np.float32)
        do, dw = desc(want, osz, abi.FP32), desc(w, ws, abi.BF16, strides=wstr)
        dx, dy = desc(x, xs, abi.BF16), desc(y, ys, abi.BF16)
        args = (A(do), A(dx), A(dw), A(do)) if op == abi.OP_FWD else (A(do), A(do), A(dw), A(dy))
        assert orc.orc_convolution(*args, A(p), op, 0) == 0, orc.orc_last_error()
        out = MmeSimTensor(osz, 5, abi.FP32, got)
        tw = MmeSimTensor(ws, 5, abi.BF16, w, strides=wstr)
        targs = (out, MmeSimTensor(xs, 5, abi.BF16, x), tw, out) if op == abi.OP_FWD else (out, out, tw, MmeSimTensor(ys, 5, abi.BF16, y))
        calc.doConvolution(*targs, cp, op)
    assert np.any(want != 0)
    assert rel_frobenius(got, want) <= TOL[abi.BF16]
