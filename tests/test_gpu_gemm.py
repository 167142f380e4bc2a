"""Batched GEMM on the GPU against the oracle (the reference's accumulation restated on the CPU).

Tolerance: relative Frobenius error of the fp32 accumulators <= 2e-3 for bf16 / fp32 operands and <= 1e-2 for fp8
operands (the bound the path's specification states); observed errors are orders of magnitude below.
"""
import numpy as np
import pytest

from intel_gaudi3_software_amd import Epilogue, MmeSimTensor, abi
from helpers import A, TOL, bf16_bits_to_f32, decode_operand, desc, random_operand, rel_frobenius

pytestmark = pytest.mark.gpu

OPS = [abi.OP_AB, abi.OP_ABT, abi.OP_ATB, abi.OP_ATBT]
TYPES = [(abi.BF16, abi.BF16, 0, 0, 0, 0), (abi.FP32, abi.FP32, 0, 0, 0, 0), (abi.FP8_143, abi.FP8_143, 7, 7, 0, 0),
         (abi.FP8_143, abi.FP8_152, 7, 15, 0, 0), (abi.FP8_152, abi.FP8_143, 20, 3, 0, 2), (abi.FP8_152, abi.FP8_152, 15, 1, 0, 0)]


def _shapes(op, M, N, K):
    ta = op in (abi.OP_ATB, abi.OP_ATBT)
    tb = op in (abi.OP_ABT, abi.OP_ATBT)
    return ([M, K] if ta else [K, M]), ([K, N] if tb else [N, K])


def _run_both(calc, orc, op, M, N, K, dtA, dtB, bA, bB, mA, mB, batch=(1, 1, 1), bcast_b=False, seed=0, device=False,
              pad=(0, 0, 0)):
    import torch
    rng = np.random.default_rng(seed)
    asz, bsz = _shapes(op, M, N, K)
    nb = int(np.prod(batch))
    bbatch = (1, 1, 1) if bcast_b else batch
    nbb = int(np.prod(bbatch))
    a_ld, b_ld, o_ld = asz[0] + pad[0], bsz[0] + pad[1], N + pad[2]
    a = random_operand(rng, dtA, a_ld * asz[1] * nb, orc, bA, mA)
    b = random_operand(rng, dtB, b_ld * bsz[1] * nbb, orc, bB, mB)
    o_ref = np.zeros(o_ld * M * nb, np.float32)
    o_gpu = np.zeros(o_ld * M * nb, np.float32)
    sa, sb, so = ([1, a_ld] if pad[0] else None), ([1, b_ld] if pad[1] else None), ([1, o_ld] if pad[2] else None)
    da = desc(a, asz + list(batch), dtA, bA, mA, sa)
    db = desc(b, bsz + list(bbatch), dtB, bB, mB, sb)
    do = desc(o_ref, [N, M] + list(batch), abi.FP32, strides=so)
    assert orc.orc_batch_gemm(A(do), A(da), A(db), op) == 0, orc.orc_last_error()
    if device:
        tt = {abi.BF16: torch.int16, abi.FP32: torch.float32}
        ta = torch.from_numpy(a.view(np.int16) if dtA == abi.BF16 else a).cuda()
        tb = torch.from_numpy(b.view(np.int16) if dtB == abi.BF16 else b).cuda()
        to = torch.zeros(o_gpu.size, dtype=torch.float32, device="cuda")
        calc.doBatchGemm(MmeSimTensor([N, M] + list(batch), 5, abi.FP32, to, strides=so),
                         MmeSimTensor(asz + list(batch), 5, dtA, ta, bA, mA, sa),
                         MmeSimTensor(bsz + list(bbatch), 5, dtB, tb, bB, mB, sb), op)
        calc.synchronize()
        o_gpu = to.cpu().numpy()
    else:
        calc.doBatchGemm(MmeSimTensor([N, M] + list(batch), 5, abi.FP32, o_gpu, strides=so),
                         MmeSimTensor(asz + list(batch), 5, dtA, a, bA, mA, sa),
                         MmeSimTensor(bsz + list(bbatch), 5, dtB, b, bB, mB, sb), op)
    return o_gpu, o_ref


@pytest.mark.parametrize("dtA,dtB,bA,bB,mA,mB", TYPES)
@pytest.mark.parametrize("op", OPS)
def test_gemm_small_ragged(calc, orc, op, dtA, dtB, bA, bB, mA, mB):
    """Sizes that are multiples of nothing: the element-wise load path, edge tiles, batch with a broadcast operand."""
    got, want = _run_both(calc, orc, op, 13, 11, 37, dtA, dtB, bA, bB, mA, mB, batch=(2, 3, 1), bcast_b=True, seed=op)
    assert rel_frobenius(got, want) <= TOL[dtA]


@pytest.mark.parametrize("dtA,dtB,bA,bB,mA,mB", TYPES)
@pytest.mark.parametrize("op", OPS)
def test_gemm_aligned_vector_path(calc, orc, op, dtA, dtB, bA, bB, mA, mB):
    """Aligned sizes: 16-byte vector loads, register transposes, several k stages, more than one tile per axis."""
    got, want = _run_both(calc, orc, op, 160, 144, 208, dtA, dtB, bA, bB, mA, mB, seed=10 + op, device=True)
    assert rel_frobenius(got, want) <= TOL[dtA]


@pytest.mark.parametrize("batch,bcast_b", [((70000, 1, 1), True), ((300, 250, 1), False), ((3, 2, 33000), True)])
def test_gemm_more_than_65535_batch_entries(calc, orc, batch, bcast_b):
    """More batch entries than one launch's grid holds along its batch axis: the call slices the slowest batch dimension
    over several launches; every entry against the oracle."""
    got, want = _run_both(calc, orc, abi.OP_AB, 3, 5, 8, abi.BF16, abi.BF16, 0, 0, 0, 0, batch=batch, bcast_b=bcast_b, seed=31, device=True)
    assert rel_frobenius(got, want) <= 1e-4
    per = 15
    blocks = np.abs(got.reshape(-1, per) - want.reshape(-1, per)).max(axis=1)
    assert np.all(blocks <= 1e-3 * max(1.0, np.abs(want).max())), int(np.argmax(blocks))


def test_gemm_strided_rows_keep_gaps(calc, orc):
    """Row pitches larger than the row (sub-views): gaps in the output keep their previous contents."""
    got, want = _run_both(calc, orc, abi.OP_AB, 9, 10, 20, abi.BF16, abi.BF16, 0, 0, 0, 0, pad=(5, 3, 2), seed=4)
    assert rel_frobenius(got, want) <= TOL[abi.BF16]
    # the oracle left the gap columns at 0 (initial value); so must the GPU path
    gaps = np.ones(got.size, bool).reshape(9, 12)
    gaps[:, :10] = False
    assert np.all(got.reshape(9, 12)[gaps] == 0)


def test_gemm_config1_bf16_512(calc, orc):
    """bf16 512^3 -> fp32, seed 1001: the CPU-runnable configuration of the baseline."""
    got, want = _run_both(calc, orc, abi.OP_AB, 512, 512, 512, abi.BF16, abi.BF16, 0, 0, 0, 0, seed=1001, device=True)
    err = rel_frobenius(got, want)
    assert err <= 2e-3
    # and both agree with the exact product of the decoded operands far inside the tolerance
    assert err <= 1e-4


def test_gemm_zero_common_dim(calc):
    out = np.full(6, 7.0, np.float32)
    calc.doBatchGemm(MmeSimTensor([3, 2], 2, abi.FP32, out), MmeSimTensor([0, 2], 2, abi.BF16, np.zeros(4, np.uint16)),
                     MmeSimTensor([3, 0], 2, abi.BF16, np.zeros(4, np.uint16)), abi.OP_AB)
    assert np.all(out == 0)


def test_fp8_bias_folding_is_exact(calc, orc):
    """Changing the exponent bias of an operand scales the result by an exact power of two."""
    import torch
    rng = np.random.default_rng(21)
    M = N = K = 64
    a = rng.integers(0, 0x78, M * K).astype(np.uint8) | (rng.integers(0, 2, M * K).astype(np.uint8) << 7)
    b = rng.integers(0, 0x78, N * K).astype(np.uint8) | (rng.integers(0, 2, N * K).astype(np.uint8) << 7)
    res = {}
    for bias in (3, 7, 11, 15):
        o = np.zeros(M * N, np.float32)
        calc.doBatchGemm(MmeSimTensor([N, M], 2, abi.FP32, o), MmeSimTensor([K, M], 2, abi.FP8_143, a, bias),
                         MmeSimTensor([N, K], 2, abi.FP8_143, b, 7), abi.OP_AB)
        res[bias] = o
    for bias in (3, 11, 15):
        assert np.array_equal(res[bias], res[7] * np.float32(2.0 ** (7 - bias)))


@pytest.mark.parametrize("M,N,K,dtA,bA,mA,dtB,bB,mB,fused", [
    (1024, 1280, 1024, abi.FP8_143, 7, 0, abi.FP8_143, 7, 0, False),      # 4 x 5 tiles, 16 stages: one workgroup per tile
    (768, 1024, 512, abi.FP8_143, 11, 1, abi.FP8_152, 15, 2, False),      # 0x7F is a number for Gaudi, exponent-31 codes likewise
    (4096, 8192, 384, abi.FP8_143, 7, 0, abi.FP8_152, 15, 0, True),       # 512 tiles, bf16 output: workgroups walk over tiles
])
def test_fp8_special_codes_found_by_the_large_tile_kernel(calc, orc, M, N, K, dtA, bA, mA, dtB, bB, mB, fused):
    """The large-tile fp8 kernels look for the codes that mean something else to the hardware while they multiply, each
    64-byte stage of a row by one of the workgroups that read it.  One such code at a time, at positions that fall to
    different workgroups, wavefronts and stages (first and last included), in A or in B: the result has to be the
    reference's, inf / NaN placement included, on the affected rows / columns and on a slab elsewhere."""
    import torch
    rng = np.random.default_rng(5)
    a0 = (rng.integers(0, 0x58, M * K).astype(np.uint8) | (rng.integers(0, 2, M * K).astype(np.uint8) << 7)).reshape(M, K)
    b0 = (rng.integers(0, 0x58, K * N).astype(np.uint8) | (rng.integers(0, 2, K * N).astype(np.uint8) << 7)).reshape(K, N)
    code_a = {0: [0x78, 0x7D, 0xF8], 1: [0x7F, 0xFF], 2: []}[mA] if dtA == abi.FP8_143 else [0x7C, 0xFD]
    code_b = ({0: [0xF8, 0x7B], 1: [0x7F], 2: []}[mB] if dtB == abi.FP8_143 else {0: [], 1: [0x7C, 0xFE], 2: [0x7D, 0xFC]}[mB])
    places = [("a", 0, 0), ("a", M - 1, K - 1), ("a", 300, 64 * 3 + 17), ("a", 129, 64 * 5 + 63), ("a", M // 2 + 1, K - 65),
              ("b", 0, 0), ("b", K - 1, N - 1), ("b", 64 * 2 + 5, 700), ("b", 64 * 4, 255), ("b", K - 64, N - 257)]
    ta, tb = torch.from_numpy(a0.ravel().copy()).cuda(), torch.from_numpy(b0.ravel().copy()).cuda()
    out = torch.zeros(M * N, dtype=torch.int16 if fused else torch.float32, device="cuda")
    X, Wt, Y = MmeSimTensor([K, M], 2, dtA, ta, bA, mA), MmeSimTensor([N, K], 2, dtB, tb, bB, mB), MmeSimTensor([N, M], 2, abi.BF16 if fused else abi.FP32, out)
    epi = Epilogue(scale_exp=-4) if fused else None

    def result():
        calc.doBatchGemm(Y, X, Wt, abi.OP_AB, epilogue=epi)
        calc.synchronize()
        r = out.cpu().numpy()
        return (bf16_bits_to_f32(r.view(np.uint16)) if fused else r).reshape(M, N)

    def expected(acc):
        if not fused:
            return acc
        codes = np.zeros(acc.size, np.uint16)
        assert orc.orc_cast_from_fp32(codes.ctypes.data, abi.BF16, 0, 0, acc.ctypes.data, acc.size, -4, None, 0, 0, 0, 0, 0, 0) == 0
        return bf16_bits_to_f32(codes)

    tol = 2e-3 if fused else 1e-4
    n_checked = 0
    for i, (which, r, c) in enumerate(places):
        codes = code_a if which == "a" else code_b
        if not codes:
            continue
        code = codes[i % len(codes)]
        a, b = a0.copy(), b0.copy()
        (a if which == "a" else b)[r, c] = code
        ta.copy_(torch.from_numpy(a.ravel()))
        tb.copy_(torch.from_numpy(b.ravel()))
        got = result()
        # rows to compare: the affected row (A) or a slab that crosses the affected column's rows (B), plus eight others
        rows = np.unique(np.concatenate([[r if which == "a" else 0], rng.choice(M, 8, replace=False)]))
        want = np.zeros(rows.size * N, np.float32)
        slab = np.ascontiguousarray(a[rows].ravel())
        assert orc.orc_batch_gemm(A(desc(want, [N, rows.size], abi.FP32)), A(desc(slab, [K, rows.size], dtA, bA, mA)), A(desc(b.ravel(), [N, K], dtB, bB, mB)),
                                  abi.OP_AB) == 0
        want = expected(want).reshape(rows.size, N)
        g = got[rows]
        assert np.array_equal(np.isnan(g), np.isnan(want)), (which, r, c, hex(code))
        inf = np.isinf(want)
        assert np.array_equal(g[inf], want[inf]), (which, r, c, hex(code))
        fin = np.isfinite(want)
        assert rel_frobenius(g[fin], want[fin]) <= tol, (which, r, c, hex(code))
        if mA == 0 and mB == 0:
            assert (~fin).any()
        n_checked += 1
    assert n_checked >= 5
    # and clean operands afterwards: the flag of the earlier calls does not stick
    ta.copy_(torch.from_numpy(a0.ravel()))
    tb.copy_(torch.from_numpy(b0.ravel()))
    got = result()
    want = np.zeros(16 * N, np.float32)
    assert orc.orc_batch_gemm(A(desc(want, [N, 16], abi.FP32)), A(desc(np.ascontiguousarray(a0[:16].ravel()), [K, 16], dtA, bA, mA)),
                              A(desc(b0.ravel(), [N, K], dtB, bB, mB)), abi.OP_AB) == 0
    assert np.isfinite(got).all() and rel_frobenius(got[:16].ravel(), expected(want)) <= tol


@pytest.mark.parametrize("policy", [abi.FP8_SPECIALS_CHECK, abi.FP8_SPECIALS_ASSUME_NONE])
@pytest.mark.parametrize("M,N,K,op,dtA,bA,dtB,bB,out_dt", [
    (4096, 4096, 3072, abi.OP_AB, abi.FP8_143, 7, abi.FP8_143, 7, abi.BF16), (4096, 4096, 3072, abi.OP_ABT, abi.FP8_143, 11, abi.FP8_152, 15, abi.FP32),
    (3072, 4096, 4096, abi.OP_AB, abi.FP8_152, 15, abi.FP8_143, 3, abi.FP8_143), (3072, 4096, 4096, abi.OP_ABT, abi.FP8_152, 17, abi.FP8_152, 12, abi.BF16)])
def test_fp8_four_wavefront_form_vs_oracle(calc, orc, policy, M, N, K, op, dtA, bA, dtB, bB, out_dt):
    """One round of tiles and a long reduction: the fp8 GEMM runs in its form with four wavefronts of 128 x 128 outputs per
    workgroup (4096 x 4096 outputs = 256 workgroups of 48 stages; 3072 x 4096 outputs = 192 workgroups of 64 stages; with
    half as many tiles or fewer the 128-row tiles take over, so this form never meets split-k).  Both operand policies (with and without the
    in-kernel look at the operand bytes), every fp8 flavour pair, B stored either way, raw fp32 and fused bf16 / fp8
    outputs: 16-row slabs from four tile rows (tile boundaries included) plus 32 random rows against the oracle, every
    column; the fused outputs also bit for bit against the oracle's cast of the GPU's own fp32 accumulators."""
    import torch
    rng = np.random.default_rng(77 + op + dtA)
    asz, bsz = _shapes(op, M, N, K)
    a = random_operand(rng, dtA, M * K, orc, bA, 0)
    b = random_operand(rng, dtB, K * N, orc, bB, 0)
    ta, tb = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()
    acc_gpu = torch.zeros(M * N, dtype=torch.float32, device="cuda")
    X, Wt = MmeSimTensor(asz, 2, dtA, ta, bA), MmeSimTensor(bsz, 2, dtB, tb, bB)
    calc.setFp8SpecialsPolicy(policy)
    try:
        calc.doBatchGemm(MmeSimTensor([N, M], 2, abi.FP32, acc_gpu), X, Wt, op)
        form = calc.lastContractionForm()
        assert form["large_tile"] and form["tile_rows"] == 256 and form["wavefronts"] == 4, form
        assert form["split_k"] == 1, form
        fused = None
        if out_dt != abi.FP32:
            fused = torch.zeros(M * N, dtype=torch.int16 if out_dt == abi.BF16 else torch.uint8, device="cuda")
            calc.doBatchGemm(MmeSimTensor([N, M], 2, out_dt, fused, 7 if out_dt == abi.FP8_143 else 0), X, Wt, op,
                             epilogue=Epilogue(scale_exp=-3, clipFp=True))
            assert calc.lastContractionForm() == form
        calc.synchronize()
    finally:
        calc.setFp8SpecialsPolicy(abi.FP8_SPECIALS_CHECK)
    got = acc_gpu.cpu().numpy().reshape(M, N)
    rows = np.concatenate([np.arange(0, 16), np.arange(3 * 256 + 120, 3 * 256 + 136), np.arange(5 * 256 - 8, 5 * 256 + 8), np.arange(M - 16, M),
                           np.sort(np.random.default_rng(3).choice(M, 32, replace=False))])
    slab = np.ascontiguousarray(a.reshape(M, K)[rows].ravel())
    want = np.zeros(rows.size * N, np.float32)
    assert orc.orc_batch_gemm(A(desc(want, [N, rows.size], abi.FP32)), A(desc(slab, [K, rows.size], dtA, bA)), A(desc(b, bsz, dtB, bB)), op) == 0
    dist = rel_frobenius(got[rows].ravel(), want)
    assert dist <= 1e-2
    assert dist <= 1e-4  # the reference's truncating tree itself sits ~1e-5 from the exact sums
    assert np.count_nonzero(got.reshape(M // 256, 256, N // 256, 256), axis=(1, 3)).min() > 256 * 256 // 2  # every tile was written
    if fused is not None:
        codes = np.zeros(M * N, np.uint16 if out_dt == abi.BF16 else np.uint8)
        flat = np.ascontiguousarray(got.ravel())
        assert orc.orc_cast_from_fp32(codes.ctypes.data, out_dt, 7 if out_dt == abi.FP8_143 else 0, 0, flat.ctypes.data, M * N, -3, None, 0, 0, 0, 1, 0, 0) == 0
        assert np.array_equal(fused.cpu().numpy().view(codes.dtype), codes)


@pytest.mark.parametrize("M,K,op,dtA,bA,mA,dtB,bB,mB,fused", [
    (3072, 3072, abi.OP_AB, abi.FP8_143, 7, 0, abi.FP8_143, 7, 0, True),      # exponent-15 codes are inf / NaN for Gaudi, 256 .. 448 for the hardware
    (3072, 3072, abi.OP_ABT, abi.FP8_143, 11, 1, abi.FP8_152, 15, 2, False),  # 0x7F is a number for Gaudi; exponent-31 codes likewise
    (3072, 3072, abi.OP_AB, abi.FP8_152, 15, 0, abi.FP8_143, 3, 0, False),    # fp8_152 in full mode is the hardware's format: its inf / NaN only end the fast conversions
    (3072, 1024, abi.OP_AB, abi.FP8_143, 7, 0, abi.FP8_143, 7, 0, True),      # a short reduction: the form with eight wavefronts, still one round of tiles
    (3072, 1024, abi.OP_ABT, abi.FP8_143, 3, 0, abi.FP8_152, 15, 1, False),
    # 4096 x 4096 outputs: all 256 compute units busy, sixteen lookers per panel of either operand
    (4096, 3072, abi.OP_AB, abi.FP8_143, 7, 0, abi.FP8_143, 7, 0, True),
    (4096, 3072, abi.OP_ABT, abi.FP8_143, 11, 1, abi.FP8_152, 15, 2, False),
])
def test_fp8_one_round_launches_recompute_tiles_with_special_codes(calc, orc, M, K, op, dtA, bA, mA, dtB, bB, mB, fused):
    """When the tiles of an fp8 GEMM make one round (3072 x 4096 outputs = 192 workgroups, 4096 x 4096 = 256), the workgroups share per operand
    panel what their looks at the operand bytes found, and a workgroup whose panels hold a code that the matrix cores read
    differently computes its tile once more from exactly decoded operands, inside the same launch.  One such code at a time,
    at positions that fall to different tiles, wavefronts and stages (first and last included), in A or in B: the affected
    rows / columns and a slab elsewhere against the oracle, inf / NaN placement included; clean operands afterwards give finite
    results again.  Both forms of the kernel (four wavefronts for the long reduction, eight for the short one)."""
    import torch
    N = 4096
    rng = np.random.default_rng(9)
    a0 = (rng.integers(0, 0x58, M * K).astype(np.uint8) | (rng.integers(0, 2, M * K).astype(np.uint8) << 7)).reshape(M, K)
    b_rows, b_cols = (N, K) if op == abi.OP_ABT else (K, N)
    b0 = (rng.integers(0, 0x58, K * N).astype(np.uint8) | (rng.integers(0, 2, K * N).astype(np.uint8) << 7)).reshape(b_rows, b_cols)
    code_a = {0: [0x78, 0x7D, 0xF8], 1: [0x7F, 0xFF], 2: [0x7F]}[mA] if dtA == abi.FP8_143 else {0: [0x7C, 0xFD], 1: [0x7C, 0xFE], 2: [0x7D]}[mA]
    code_b = {0: [0xF8, 0x7B], 1: [0x7F], 2: [0x7F]}[mB] if dtB == abi.FP8_143 else {0: [0x7C], 1: [0x7C, 0xFE], 2: [0x7D, 0xFC]}[mB]
    # (which, f index, k index): rows of A / columns of B in different tiles and quarters of a tile, k in different stages
    places = [("a", 0, 0), ("a", M - 1, K - 1), ("a", 300, 64 * 3 + 17), ("a", 5 * 256 + 129, 64 * (K // 150) + 63), ("a", 7 * 256 + 70, K - 65),
              ("b", 0, 0), ("b", N - 1, K - 1), ("b", 700, 64 * 2 + 5), ("b", 9 * 256 + 200, 64 * (K // 100)), ("b", 13 * 256 + 64, K - 64)]
    asz, bsz = _shapes(op, M, N, K)
    ta, tb = torch.from_numpy(a0.ravel().copy()).cuda(), torch.from_numpy(b0.ravel().copy()).cuda()
    out = torch.zeros(M * N, dtype=torch.int16 if fused else torch.float32, device="cuda")
    X, Wt, Y = MmeSimTensor(asz, 2, dtA, ta, bA, mA), MmeSimTensor(bsz, 2, dtB, tb, bB, mB), MmeSimTensor([N, M], 2, abi.BF16 if fused else abi.FP32, out)
    epi = Epilogue(scale_exp=-4) if fused else None

    def result():
        calc.doBatchGemm(Y, X, Wt, op, epilogue=epi)
        form = calc.lastContractionForm()
        assert form["large_tile"] and form["wavefronts"] == (4 if K >= 3072 else 8) and form["split_k"] == 1 and form["tile_rows"] == 256, form
        calc.synchronize()
        r = out.cpu().numpy()
        return (bf16_bits_to_f32(r.view(np.uint16)) if fused else r).reshape(M, N)

    def expected(acc):
        if not fused:
            return acc
        codes = np.zeros(acc.size, np.uint16)
        assert orc.orc_cast_from_fp32(codes.ctypes.data, abi.BF16, 0, 0, acc.ctypes.data, acc.size, -4, None, 0, 0, 0, 0, 0, 0) == 0
        return bf16_bits_to_f32(codes)

    def reference_rows(a, b, rows):
        want = np.zeros(rows.size * N, np.float32)
        slab = np.ascontiguousarray(a[rows].ravel())
        assert orc.orc_batch_gemm(A(desc(want, [N, rows.size], abi.FP32)), A(desc(slab, [K, rows.size], dtA, bA, mA)), A(desc(b.ravel(), bsz, dtB, bB, mB)), op) == 0
        return expected(want).reshape(rows.size, N)

    tol = 2e-3 if fused else 1e-4
    n_checked = n_nonfinite = 0
    for i, (which, fi, ki) in enumerate(places):
        codes = code_a if which == "a" else code_b
        code = codes[i % len(codes)]
        a, b = a0.copy(), b0.copy()
        if which == "a":
            a[fi, ki] = code
        elif op == abi.OP_ABT:
            b[fi, ki] = code
        else:
            b[ki, fi] = code
        ta.copy_(torch.from_numpy(a.ravel()))
        tb.copy_(torch.from_numpy(b.ravel()))
        got = result()
        # the affected row (A), or rows of three different tile rows that all cross the affected column (B), plus six others
        rows = np.unique(np.concatenate([[fi] if which == "a" else [1, M // 2 + 3, M - 2], rng.choice(M, 6, replace=False)]))
        want = reference_rows(a, b, rows)
        g = got[rows]
        assert np.array_equal(np.isnan(g), np.isnan(want)), (which, fi, ki, hex(code))
        inf = np.isinf(want)
        assert np.array_equal(g[inf], want[inf]), (which, fi, ki, hex(code))
        fin = np.isfinite(want)
        assert rel_frobenius(g[fin], want[fin]) <= tol, (which, fi, ki, hex(code))
        n_nonfinite += int((~fin).any())
        n_checked += 1
    assert n_checked == len(places)
    if mA == 0 or mB == 0:
        assert n_nonfinite >= 3
    ta.copy_(torch.from_numpy(a0.ravel()))
    tb.copy_(torch.from_numpy(b0.ravel()))
    got = result()
    rows = np.arange(16)
    assert np.isfinite(got).all() and rel_frobenius(got[rows].ravel(), reference_rows(a0, b0, rows).ravel()) <= tol


@pytest.mark.parametrize("K", [3072, 1024])
def test_fp8_one_round_launch_with_batches_settles_special_codes_per_batch_element(calc, orc, K):
    """Two batch elements of 1536 x 4096 outputs (2 x 96 tiles: one round), A per batch element, B shared: the panel words in
    which the workgroups share their finds are kept per batch element.  A special code in batch element 1 of A, and one in
    the shared B: the first changes rows of batch element 1 only, the second columns of both; everything against the oracle."""
    import torch
    M, N = 1536, 4096
    rng = np.random.default_rng(31)
    a = (rng.integers(0, 0x58, 2 * M * K).astype(np.uint8) | (rng.integers(0, 2, 2 * M * K).astype(np.uint8) << 7)).reshape(2, M, K)
    b = (rng.integers(0, 0x58, K * N).astype(np.uint8) | (rng.integers(0, 2, K * N).astype(np.uint8) << 7)).reshape(K, N)
    a[1, 700, K - 3] = 0x78      # +inf for Gaudi's fp8_143 in full mode
    b[64 * 5 + 9, 2049] = 0x7D   # NaN
    ta, tb = torch.from_numpy(a.ravel().copy()).cuda(), torch.from_numpy(b.ravel().copy()).cuda()
    out = torch.zeros(2 * M * N, dtype=torch.float32, device="cuda")
    calc.doBatchGemm(MmeSimTensor([N, M, 2, 1, 1], 5, abi.FP32, out), MmeSimTensor([K, M, 2, 1, 1], 5, abi.FP8_143, ta, 7),
                     MmeSimTensor([N, K, 1, 1, 1], 5, abi.FP8_143, tb, 7), abi.OP_AB)
    form = calc.lastContractionForm()
    assert form["large_tile"] and form["tile_rows"] == 256 and form["split_k"] == 1 and form["wavefronts"] == (4 if K >= 3072 else 8), form
    calc.synchronize()
    got = out.cpu().numpy().reshape(2, M, N)
    rows = np.array([0, 5, 255, 256, 699, 700, 701, 1000, M - 1])
    for bz in range(2):
        want = np.zeros(rows.size * N, np.float32)
        slab = np.ascontiguousarray(a[bz][rows].ravel())
        assert orc.orc_batch_gemm(A(desc(want, [N, rows.size], abi.FP32)), A(desc(slab, [K, rows.size], abi.FP8_143, 7)), A(desc(b.ravel(), [N, K], abi.FP8_143, 7)), abi.OP_AB) == 0
        want = want.reshape(rows.size, N)
        g = got[bz][rows]
        assert np.array_equal(np.isnan(g), np.isnan(want)) and np.array_equal(np.isinf(g), np.isinf(want)), bz
        fin = np.isfinite(want)
        assert np.array_equal(g[~fin & ~np.isnan(want)], want[~fin & ~np.isnan(want)])
        assert rel_frobenius(g[fin], want[fin]) <= 1e-4
        # column 2049 is NaN in every row of both batch elements, row 700 is not finite in batch element 1 only
        assert np.isnan(got[bz][:, 2049]).all()
        assert np.isfinite(np.delete(got[bz], 2049, axis=1)[np.arange(M) != 700]).all()
    assert np.isfinite(np.delete(got[0][700], 2049)).all() and not np.isfinite(np.delete(got[1][700], 2049)).any()


def test_fp8_short_reductions_keep_eight_wavefronts(calc):
    """Below 48 stages per workgroup, or with more tiles than one round, the form with eight wavefronts stays."""
    import torch
    for M, N, K, waves in ((4096, 4096, 1024, 8), (4096, 4096, 4096, 4), (8192, 8192, 4096, 8), (512, 512, 512, 8)):
        ta, tb = torch.zeros(M * K, dtype=torch.uint8, device="cuda"), torch.zeros(K * N, dtype=torch.uint8, device="cuda")
        out = torch.zeros(M * N, dtype=torch.int16, device="cuda")
        calc.doBatchGemm(MmeSimTensor([N, M], 2, abi.BF16, out), MmeSimTensor([K, M], 2, abi.FP8_143, ta, 7), MmeSimTensor([N, K], 2, abi.FP8_143, tb, 7),
                         abi.OP_AB, epilogue=Epilogue(scale_exp=-2, clipFp=True))
        calc.synchronize()
        form = calc.lastContractionForm()
        assert form["large_tile"] and form["wavefronts"] == waves, (M, N, K, form)


def test_fp8_special_codes_take_exact_path(calc, orc):
    """fp8_143 in full inf/nan mode: exponent-15 codes are inf / NaN for Gaudi and finite for the hardware's e4m3.
    The library must notice them and still agree with the reference (NaN / inf placement included)."""
    rng = np.random.default_rng(22)
    M, N, K = 48, 40, 96
    a = rng.integers(0, 0x70, M * K).astype(np.uint8)
    b = rng.integers(0, 0x70, N * K).astype(np.uint8)
    a[5 * K + 3] = 0x78   # +inf in row 5
    a[9 * K + 1] = 0x7D   # NaN in row 9
    b[7 * N + 2] = 0xF8   # -inf in column 2 (k = 7)
    want = np.zeros(M * N, np.float32)
    da, db, do = desc(a, [K, M], abi.FP8_143, 7), desc(b, [N, K], abi.FP8_143, 7), desc(want, [N, M], abi.FP32)
    assert orc.orc_batch_gemm(A(do), A(da), A(db), abi.OP_AB) == 0
    got = np.zeros(M * N, np.float32)
    calc.doBatchGemm(MmeSimTensor([N, M], 2, abi.FP32, got), MmeSimTensor([K, M], 2, abi.FP8_143, a, 7),
                     MmeSimTensor([N, K], 2, abi.FP8_143, b, 7), abi.OP_AB)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    assert np.array_equal(np.isinf(got), np.isinf(want))
    fin = np.isfinite(want)
    assert np.array_equal(np.sign(got[~fin & ~np.isnan(want)]), np.sign(want[~fin & ~np.isnan(want)]))
    assert rel_frobenius(got[fin], want[fin]) <= 1e-2
    assert np.isnan(want).any() and np.isinf(want).any()


@pytest.mark.parametrize("out_dt,out_bias", [(abi.BF16, 0), (abi.FP8_143, 7), (abi.FP8_152, 15), (abi.FP32, 0)])
def test_fused_epilogue_equals_gemm_then_cast(calc, orc, out_dt, out_bias):
    """Fused descale + relu + cast == (fp32 GEMM on the GPU) -> oracle cast of the same accumulators, bit for bit."""
    import torch
    rng = np.random.default_rng(31)
    M, N, K = 96, 80, 128
    a = random_operand(rng, abi.FP8_143, M * K, orc, 7)
    b = random_operand(rng, abi.FP8_152, N * K, orc, 15, scale=0.05)
    col = rng.integers(-3, 4, N).astype(np.int32)
    ta, tb = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()
    acc = torch.zeros(M * N, dtype=torch.float32, device="cuda")
    X = MmeSimTensor([K, M], 2, abi.FP8_143, ta, 7)
    W = MmeSimTensor([N, K], 2, abi.FP8_152, tb, 15)
    calc.doBatchGemm(MmeSimTensor([N, M], 2, abi.FP32, acc), X, W, abi.OP_AB)
    td = {abi.BF16: torch.int16, abi.FP32: torch.float32}.get(out_dt, torch.uint8)
    out = torch.zeros(M * N, dtype=td, device="cuda")
    epi = Epilogue(scale_exp=-2, col_scale_exp=torch.from_numpy(col).cuda(), relu=True, clipFp=True)
    calc.doBatchGemm(MmeSimTensor([N, M], 2, out_dt, out, out_bias), X, W, abi.OP_AB, epilogue=epi)
    calc.synchronize()
    acc_h = acc.cpu().numpy()
    want = np.zeros(M * N, abi.DTYPE_NUMPY[out_dt] if out_dt != abi.FP32 else np.uint32)
    assert orc.orc_cast_from_fp32(want.ctypes.data, out_dt, out_bias, 0, acc_h.ctypes.data, M * N, -2, col.ctypes.data, N, 1,
                                  0, 1, 0, 0) == 0
    got = out.cpu().numpy()
    got = got.view(np.uint16) if out_dt == abi.BF16 else (got.view(np.uint32) if out_dt == abi.FP32 else got)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("out_dt,out_bias,rm", [(abi.BF16, 0, 4), (abi.FP8_143, 7, 4), (abi.FP8_152, 15, 7), (abi.FP16, 15, 4)])
@pytest.mark.parametrize("M,N,K,ld", [(96, 80, 128, 80), (256, 256, 512, 256), (70, 48, 64, 56)])
def test_fused_epilogue_with_stochastic_rounding(orc, out_dt, out_bias, rm, M, N, K, ld):
    """A fused epilogue that rounds stochastically == the reference's sequence: contraction -> power-of-two scales and relu
    -> doActivation with the calculator's LFSR registers (element i of the flat output takes register i % L after i / L
    steps).  Two contractions in a row on each side (the registers carry over), on a small shape, one that takes the
    large-tile kernel and one whose output rows have a pitch (the gaps are converted like the reference's zero-filled
    accumulator tensor): the GPU's fused result against the oracle's doActivation of the GPU's own fp32 results."""
    import torch
    from intel_gaudi3_software_amd import HipCalculator
    rng = np.random.default_rng(M + rm)
    lfsr = (np.arange(256, dtype=np.uint32) * 2654435761 + 977).astype(np.uint32)
    poly = 0x9C35
    fused_calc = HipCalculator(lfsrNumRegs=256, lfsr=lfsr, polynomial=poly)
    plain_calc = HipCalculator(lfsrNumRegs=256, lfsr=lfsr, polynomial=poly)
    regs = lfsr.copy()   # the oracle's registers, carried from call to call
    td = {abi.BF16: torch.int16, abi.FP16: torch.int16}.get(out_dt, torch.uint8)
    col = rng.integers(-2, 3, N).astype(np.int32)
    so = None if ld == N else [1, ld]
    try:
        for call in range(2):
            a = random_operand(rng, abi.FP8_143, M * K, orc, 7)
            b = random_operand(rng, abi.FP8_152, N * K, orc, 15, scale=0.05)
            X = MmeSimTensor([K, M], 2, abi.FP8_143, torch.from_numpy(a).cuda(), 7)
            W = MmeSimTensor([N, K], 2, abi.FP8_152, torch.from_numpy(b).cuda(), 15)
            # (a sentinel in every byte: with a stochastic mode the gaps between strided rows are converted too and must come
            # out as the code of zero, as the reference's doActivation over the tensor's span leaves them)
            out = torch.full((M * ld,), 0x55, dtype=td, device="cuda")
            epi = Epilogue(scale_exp=-1, col_scale_exp=torch.from_numpy(col).cuda(), relu=bool(call), rm=rm, clipFp=True)
            fused_calc.doBatchGemm(MmeSimTensor([N, M], 2, out_dt, out, out_bias, strides=so), X, W, abi.OP_AB, epilogue=epi)
            fused_calc.synchronize()
            # the same scaled (and rectified) fp32 values, then the oracle's doActivation with the registers so far
            acc = torch.zeros(M * ld, dtype=torch.float32, device="cuda")
            plain = Epilogue(scale_exp=-1, col_scale_exp=torch.from_numpy(col).cuda(), relu=bool(call))
            plain_calc.doBatchGemm(MmeSimTensor([N, M], 2, abi.FP32, acc, strides=so), X, W, abi.OP_AB, epilogue=plain)
            plain_calc.synchronize()
            acc_h = acc.cpu().numpy()
            want = np.zeros(M * ld, abi.DTYPE_NUMPY[out_dt])
            d_o, d_a = desc(want, [N, M], out_dt, out_bias, strides=so), desc(acc_h, [N, M], abi.FP32, strides=so)
            assert orc.orc_activation(A(d_o), A(d_a), 0, rm, 1, 0, 0, 0, regs.ctypes.data, poly) == 0, orc.orc_last_error()
            got = out.cpu().numpy().view(want.dtype)
            assert np.array_equal(got, want), (call, int(np.argmax(got != want)))
            assert np.any(want != 0)
    finally:
        fused_calc.close()
        plain_calc.close()


def test_gemm_linearity_large(calc, orc):
    """Size-independent property at a large shape (2048 x 1024 x 4096 fp8): doubling A via its exponent bias doubles
    the result exactly; a 64-row slab agrees with the oracle."""
    import torch
    rng = np.random.default_rng(41)
    M, N, K = 2048, 1024, 4096
    a = random_operand(rng, abi.FP8_143, M * K, orc, 7, scale=40.0)
    b = random_operand(rng, abi.FP8_143, N * K, orc, 7, scale=40.0)
    ta, tb = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()
    o1 = torch.zeros(M * N, dtype=torch.float32, device="cuda")
    o2 = torch.zeros(M * N, dtype=torch.float32, device="cuda")
    calc.doBatchGemm(MmeSimTensor([N, M], 2, abi.FP32, o1), MmeSimTensor([K, M], 2, abi.FP8_143, ta, 7),
                     MmeSimTensor([N, K], 2, abi.FP8_143, tb, 7), abi.OP_AB)
    calc.doBatchGemm(MmeSimTensor([N, M], 2, abi.FP32, o2), MmeSimTensor([K, M], 2, abi.FP8_143, ta, 3),
                     MmeSimTensor([N, K], 2, abi.FP8_143, tb, 11), abi.OP_AB)
    calc.synchronize()
    assert torch.equal(o1, o2)  # 2^(7-3) * 2^(7-11) = 1
    rows = 64
    want = np.zeros(rows * N, np.float32)
    da, db, do = desc(a, [K, rows], abi.FP8_143, 7), desc(b, [N, K], abi.FP8_143, 7), desc(want, [N, rows], abi.FP32)
    assert orc.orc_batch_gemm(A(do), A(da), A(db), abi.OP_AB) == 0
    assert rel_frobenius(o1.cpu().numpy()[:rows * N], want) <= 1e-2


# ---- the large-aligned fp8 kernel (256 x 256 tiles, LDS DMA ring, transposed LDS reads) ---------------------------------
@pytest.mark.parametrize("dtA,dtB,bA,bB", [(abi.FP8_143, abi.FP8_143, 7, 7), (abi.FP8_143, abi.FP8_152, 7, 15),
                                           (abi.FP8_152, abi.FP8_143, 15, 11), (abi.FP8_152, abi.FP8_152, 20, 15)])
@pytest.mark.parametrize("op", OPS)
def test_fp8_fast_kernel_vs_oracle(calc, orc, op, dtA, dtB, bA, bB):
    """Shapes that take the fast path (M, N multiples of 256, K multiple of 128 and >= 384), every fp8 flavour pair,
    all four layouts, batch of 2 with B broadcast; fp32 accumulators against the oracle."""
    got, want = _run_both(calc, orc, op, 256, 512, 384, dtA, dtB, bA, bB, 0, 0, batch=(2, 1, 1), bcast_b=True, seed=50 + op,
                          device=True)
    assert rel_frobenius(got, want) <= 1e-2
    assert rel_frobenius(got, want) <= 1e-4  # the reference's truncating tree itself sits ~1e-5 from the exact sums


@pytest.mark.parametrize("a_transposed", [False, True])
def test_fp8_fast_kernel_every_k_position(calc, orc, a_transposed):
    """One-hot operands walk a single product through every k position and every tile coordinate: catches any
    fragment / swizzle / transposed-read mix-up that random data could average out.  A as M x K rows or stored K x M."""
    import torch
    M, N, K = 256, 256, 512
    one = 0x38  # 1.0 in fp8_143 bias 7
    a = np.zeros((M, K), np.uint8)
    b = np.zeros((K, N), np.uint8)
    rng = np.random.default_rng(3)
    perm_m = rng.permutation(M)
    for k in range(K):
        a[perm_m[k % M], k] = one
        b[k, (k * 7 + 3) % N] = 0x40 if k % 2 else one   # 2.0 / 1.0
    want = (a == one).astype(np.float64) @ np.where(b == 0x40, 2.0, (b == one) * 1.0)
    a_stored = np.ascontiguousarray(a.T) if a_transposed else a
    ta, tb = torch.from_numpy(a_stored.ravel()).cuda(), torch.from_numpy(b.ravel()).cuda()
    out = torch.zeros(M * N, dtype=torch.float32, device="cuda")
    calc.doBatchGemm(MmeSimTensor([N, M], 2, abi.FP32, out), MmeSimTensor([M, K] if a_transposed else [K, M], 2, abi.FP8_143, ta, 7),
                     MmeSimTensor([N, K], 2, abi.FP8_143, tb, 7), abi.OP_ATB if a_transposed else abi.OP_AB)
    calc.synchronize()
    assert np.array_equal(out.cpu().numpy().reshape(M, N).astype(np.float64), want)


def test_fp8_fast_kernel_fused_epilogue_bit_exact(calc, orc):
    """bf16 / fp8 outputs of the fast kernel == its own fp32 accumulators pushed through the oracle cast."""
    import torch
    rng = np.random.default_rng(61)
    M, N, K = 256, 256, 384
    a = random_operand(rng, abi.FP8_143, M * K, orc, 7)
    b = random_operand(rng, abi.FP8_152, N * K, orc, 15, scale=0.05)
    col = rng.integers(-3, 4, N).astype(np.int32)
    ta, tb = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()
    X, W = MmeSimTensor([K, M], 2, abi.FP8_143, ta, 7), MmeSimTensor([N, K], 2, abi.FP8_152, tb, 15)
    acc = torch.zeros(M * N, dtype=torch.float32, device="cuda")
    calc.doBatchGemm(MmeSimTensor([N, M], 2, abi.FP32, acc), X, W, abi.OP_AB)
    for out_dt, out_bias, td in [(abi.BF16, 0, torch.int16), (abi.FP8_143, 7, torch.uint8)]:
        out = torch.zeros(M * N, dtype=td, device="cuda")
        epi = Epilogue(scale_exp=3, col_scale_exp=torch.from_numpy(col).cuda(), relu=True, clipFp=True)
        calc.doBatchGemm(MmeSimTensor([N, M], 2, out_dt, out, out_bias), X, W, abi.OP_AB, epilogue=epi)
        calc.synchronize()
        acc_h = acc.cpu().numpy()
        want = np.zeros(M * N, abi.DTYPE_NUMPY[out_dt])
        assert orc.orc_cast_from_fp32(want.ctypes.data, out_dt, out_bias, 0, acc_h.ctypes.data, M * N, 3, col.ctypes.data, N, 1, 0,
                                      1, 0, 0) == 0
        got = out.cpu().numpy()
        assert np.array_equal(got.view(want.dtype), want)


@pytest.mark.parametrize("clip", [False, True])
def test_fp8_fast_kernel_epilogue_overflow_takes_exact_conversion(calc, orc, clip):
    """A descale that pushes part of the accumulators beyond the bf16 range: those blocks leave the hardware-convert path
    for the exact converter (inf without clipping, the largest normal with it); bit-exact against the oracle cast."""
    import torch
    rng = np.random.default_rng(67)
    M, N, K = 256, 256, 384
    a = random_operand(rng, abi.FP8_143, M * K, orc, 7)
    b = random_operand(rng, abi.FP8_143, N * K, orc, 7)
    ta, tb = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()
    X, W = MmeSimTensor([K, M], 2, abi.FP8_143, ta, 7), MmeSimTensor([N, K], 2, abi.FP8_143, tb, 7)
    acc = torch.zeros(M * N, dtype=torch.float32, device="cuda")
    calc.doBatchGemm(MmeSimTensor([N, M], 2, abi.FP32, acc), X, W, abi.OP_AB)
    # per-column exponents: most columns stay finite, some overflow to inf in fp32, some only in bf16
    col = np.zeros(N, np.int32)
    col[::7] = 126
    col[3::11] = 124
    out = torch.zeros(M * N, dtype=torch.int16, device="cuda")
    epi = Epilogue(scale_exp=0, col_scale_exp=torch.from_numpy(col).cuda(), clipFp=clip)
    calc.doBatchGemm(MmeSimTensor([N, M], 2, abi.BF16, out), X, W, abi.OP_AB, epilogue=epi)
    calc.synchronize()
    acc_h = acc.cpu().numpy()
    want = np.zeros(M * N, np.uint16)
    assert orc.orc_cast_from_fp32(want.ctypes.data, abi.BF16, 0, 0, acc_h.ctypes.data, M * N, 0, col.ctypes.data, N, 0, 0, int(clip), 0, 0) == 0
    got = out.cpu().numpy().view(np.uint16)
    assert np.array_equal(got, want)
    assert (np.any((want & 0x7FFF) == 0x7F7F) if clip else np.any((want & 0x7FFF) == 0x7F80))


@pytest.mark.parametrize("policy", [abi.FP8_SPECIALS_CHECK, abi.FP8_SPECIALS_ASSUME_NONE])
@pytest.mark.parametrize("clip", [False, True])
@pytest.mark.parametrize("scale_exp", [84, 88, 92])
def test_fp8_152_operands_of_largest_magnitude_with_a_large_descale(calc, orc, scale_exp, clip, policy):
    """fp8_152 x fp8_152 with every operand at the largest finite magnitude (57344, about 2^15.8): products reach 2^31.6 and
    sums over K = 4096 2^43.6, so a power-of-two factor of 2^84 and more takes them beyond the fp32 and bf16 ranges.  The
    host may then neither promise the epilogue finite values nor hand the factor to the matrix instruction: the fused bf16
    output must equal the oracle's cast of the GPU's own fp32 accumulators, bit for bit, under both policies for special codes."""
    import torch
    M, N, K = 256, 256, 4096
    rng = np.random.default_rng(scale_exp)
    a = np.where(rng.random(M * K) < 0.5, 0x7B, 0xFB).astype(np.uint8)
    b = np.full(N * K, 0x7B, np.uint8)
    # rows whose signs cancel down to a finite result, rows that do not
    a.reshape(M, K)[::3] = 0x7B
    ta, tb = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()
    X, W = MmeSimTensor([K, M], 2, abi.FP8_152, ta, 15), MmeSimTensor([N, K], 2, abi.FP8_152, tb, 15)
    acc = torch.zeros(M * N, dtype=torch.float32, device="cuda")
    out = torch.zeros(M * N, dtype=torch.int16, device="cuda")
    calc.setFp8SpecialsPolicy(policy)
    try:
        calc.doBatchGemm(MmeSimTensor([N, M], 2, abi.FP32, acc), X, W, abi.OP_AB)
        calc.doBatchGemm(MmeSimTensor([N, M], 2, abi.BF16, out), X, W, abi.OP_AB, epilogue=Epilogue(scale_exp=scale_exp, clipFp=clip))
        assert calc.lastContractionForm()["large_tile"]
        calc.synchronize()
    finally:
        calc.setFp8SpecialsPolicy(abi.FP8_SPECIALS_CHECK)
    acc_h = acc.cpu().numpy()
    assert np.isfinite(acc_h).all() and np.abs(acc_h).max() == np.float32(57344.0 * 57344.0 * K)
    want = np.zeros(M * N, np.uint16)
    assert orc.orc_cast_from_fp32(want.ctypes.data, abi.BF16, 0, 0, acc_h.ctypes.data, M * N, scale_exp, None, 0, 0, 0, int(clip), 0, 0) == 0
    got = out.cpu().numpy().view(np.uint16)
    assert np.array_equal(got, want), int(np.argmax(got != want))
    # (2^84 leaves the largest sum, 49 * 2^122, just inside the bf16 range; 2^88 and 2^92 do not)
    # (there the product with the factor is already infinite in fp32, which clipFp alone leaves infinite)
    assert scale_exp < 85 or np.any((want & 0x7FFF) == 0x7F80)
    assert np.any((want & 0x7FFF) < 0x7F00)  # rows whose signs cancel stay finite


@pytest.mark.parametrize("clip", [False, True])
@pytest.mark.parametrize("out_dt,out_bias", [(abi.FP8_143, 7), (abi.FP8_143, 3), (abi.FP8_143, 11), (abi.FP8_152, 15), (abi.FP8_152, 20),
                                             (abi.FP8_152, 9)])
def test_fp8_fast_kernel_fp8_output_hardware_convert_bit_exact(calc, orc, out_dt, out_bias, clip):
    """fp8 outputs of the large-tile kernel for several exponent biases, clipping on and off.  Per-column descales spread
    the accumulators over the whole target range: denormal codes, rounding to zero, overflow to the format's inf (or its
    largest normal), fp32 overflow to inf (those blocks leave the hardware converter).  Bit-exact against the oracle cast of
    the kernel's own fp32 accumulators."""
    import torch
    rng = np.random.default_rng(71)
    M, N, K = 256, 256, 384
    a = random_operand(rng, abi.FP8_143, M * K, orc, 7)
    b = random_operand(rng, abi.FP8_143, N * K, orc, 7)
    ta, tb = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()
    X, W = MmeSimTensor([K, M], 2, abi.FP8_143, ta, 7), MmeSimTensor([N, K], 2, abi.FP8_143, tb, 7)
    acc = torch.zeros(M * N, dtype=torch.float32, device="cuda")
    calc.doBatchGemm(MmeSimTensor([N, M], 2, abi.FP32, acc), X, W, abi.OP_AB)
    col = rng.integers(-40, 24, N).astype(np.int32)
    col[::13] = 126
    out = torch.zeros(M * N, dtype=torch.uint8, device="cuda")
    epi = Epilogue(scale_exp=0, col_scale_exp=torch.from_numpy(col).cuda(), clipFp=clip)
    calc.doBatchGemm(MmeSimTensor([N, M], 2, out_dt, out, out_bias), X, W, abi.OP_AB, epilogue=epi)
    calc.synchronize()
    acc_h = acc.cpu().numpy()
    want = np.zeros(M * N, np.uint8)
    assert orc.orc_cast_from_fp32(want.ctypes.data, out_dt, out_bias, 0, acc_h.ctypes.data, M * N, 0, col.ctypes.data, N, 0, 0, int(clip), 0,
                                  0) == 0
    got = out.cpu().numpy()
    assert np.array_equal(got, want)
    man = 3 if out_dt == abi.FP8_143 else 2
    mag = want & 0x7F
    assert np.any((mag > 0) & (mag < (1 << man))) and np.any(mag == 0) and np.any(mag >= (0x7F >> man << man) - 1)


@pytest.mark.parametrize("op", [abi.OP_AB, abi.OP_ABT, abi.OP_ATB, abi.OP_ATBT])
def test_bf16_fast_kernel_vs_oracle(calc, orc, op):
    """bf16 shapes that take the large-tile kernel (M, N multiples of 256, K multiple of 64 and >= 192), all four layouts,
    batch of 2 with B broadcast; fp32 accumulators against the oracle."""
    got, want = _run_both(calc, orc, op, 256, 512, 320, abi.BF16, abi.BF16, 0, 0, 0, 0, batch=(2, 1, 1), bcast_b=True, seed=80 + op,
                          device=True)
    assert rel_frobenius(got, want) <= 2e-3
    assert rel_frobenius(got, want) <= 1e-4


@pytest.mark.parametrize("b_kc", [False, True])
def test_bf16_fast_kernel_every_k_position(calc, orc, b_kc):
    """One-hot bf16 operands walk a single product through every k position and tile coordinate of the large-tile kernel:
    the k order of the transposing reads of an n-contiguous B must match the k-contiguous reads of A."""
    import torch
    from helpers import to_bf16_bits
    M, N, K = 256, 256, 384
    a = np.zeros((M, K), np.float32)
    b = np.zeros((K, N), np.float32)
    rng = np.random.default_rng(5)
    perm_m = rng.permutation(M)
    for k in range(K):
        a[perm_m[k % M], k] = 1.0 + (k % 5)
        b[k, (k * 11 + 2) % N] = 2.0 if k % 2 else 1.0
    want = a.astype(np.float64) @ b.astype(np.float64)
    bmat = b.T.copy() if b_kc else b
    ta = torch.from_numpy(to_bf16_bits(a.ravel()).view(np.int16)).cuda()
    tb = torch.from_numpy(to_bf16_bits(bmat.ravel()).view(np.int16)).cuda()
    out = torch.zeros(M * N, dtype=torch.float32, device="cuda")
    calc.doBatchGemm(MmeSimTensor([N, M], 2, abi.FP32, out), MmeSimTensor([K, M], 2, abi.BF16, ta),
                     MmeSimTensor([K, N] if b_kc else [N, K], 2, abi.BF16, tb), abi.OP_ABT if b_kc else abi.OP_AB)
    calc.synchronize()
    assert np.array_equal(out.cpu().numpy().reshape(M, N).astype(np.float64), want)


# ---- the large-tile kernel on shapes that are not whole tiles: any M from 64 (A's rows along the tile's rows), N a multiple of 16
RAGGED_FAST = [(300, 400, 384, (0, 0, 16), (1, 1, 1)), (77, 144, 2048, (0, 0, 0), (1, 1, 1)), (520, 272, 512, (0, 0, 0), (2, 1, 1))]


@pytest.mark.parametrize("dtA,dtB,bA,bB", [(abi.FP8_143, abi.FP8_143, 7, 7), (abi.FP8_152, abi.FP8_143, 15, 11), (abi.BF16, abi.BF16, 0, 0)])
@pytest.mark.parametrize("op", [abi.OP_AB, abi.OP_ABT])
@pytest.mark.parametrize("M,N,K,pad,batch", RAGGED_FAST)
def test_fast_kernel_partial_row_and_column_tiles(calc, orc, op, dtA, dtB, bA, bB, M, N, K, pad, batch):
    """Loads of a partial tile stay inside the operands and its stores inside the output: the gap columns of a padded output
    keep their zeros (the comparison covers them), a long reduction over few tiles is split over k."""
    got, want = _run_both(calc, orc, op, M, N, K, dtA, dtB, bA, bB, 0, 0, batch=batch, bcast_b=batch != (1, 1, 1), seed=90 + op, device=True,
                          pad=pad)
    assert rel_frobenius(got, want) <= 1e-4
    ld, nb = N + pad[2], int(np.prod(batch))
    assert not got.reshape(M * nb, ld)[:, N:].any(), "gap columns were written"


@pytest.mark.parametrize("out_dt,out_bias", [(abi.BF16, 0), (abi.FP8_143, 7), (abi.FP32, 0)])
def test_fast_kernel_partial_tiles_fused_epilogue_bit_exact(calc, orc, out_dt, out_bias):
    """Per-column scale exponents, descale, relu and the output cast on partial tiles: the fused output equals the oracle's
    cast of the same kernel's fp32 accumulators, bit for bit."""
    import torch
    rng = np.random.default_rng(32)
    M, N, K = 300, 400, 384
    a = random_operand(rng, abi.FP8_143, M * K, orc, 7)
    b = random_operand(rng, abi.FP8_152, N * K, orc, 15, scale=0.05)
    col = rng.integers(-3, 4, N).astype(np.int32)
    ta, tb = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()
    acc = torch.zeros(M * N, dtype=torch.float32, device="cuda")
    X = MmeSimTensor([K, M], 2, abi.FP8_143, ta, 7)
    W = MmeSimTensor([N, K], 2, abi.FP8_152, tb, 15)
    calc.doBatchGemm(MmeSimTensor([N, M], 2, abi.FP32, acc), X, W, abi.OP_AB)
    td = {abi.BF16: torch.int16, abi.FP32: torch.float32}.get(out_dt, torch.uint8)
    out = torch.zeros(M * N, dtype=td, device="cuda")
    epi = Epilogue(scale_exp=-2, col_scale_exp=torch.from_numpy(col).cuda(), relu=True, clipFp=True)
    calc.doBatchGemm(MmeSimTensor([N, M], 2, out_dt, out, out_bias), X, W, abi.OP_AB, epilogue=epi)
    calc.synchronize()
    acc_h = acc.cpu().numpy()
    want = np.zeros(M * N, abi.DTYPE_NUMPY[out_dt] if out_dt != abi.FP32 else np.uint32)
    assert orc.orc_cast_from_fp32(want.ctypes.data, out_dt, out_bias, 0, acc_h.ctypes.data, M * N, -2, col.ctypes.data, N, 1,
                                  0, 1, 0, 0) == 0
    got = out.cpu().numpy()
    got = got.view(np.uint16) if out_dt == abi.BF16 else (got.view(np.uint32) if out_dt == abi.FP32 else got)
    assert np.array_equal(got, want)


# ---- fp32 operands on the bf16 matrix cores: three bf16 parts per value, six cross products (plain GEMMs from 2^26 multiply-adds)
@pytest.mark.parametrize("op", OPS)
def test_fp32_three_part_path_vs_oracle_and_float64(calc, orc, op):
    """An aligned shape (the large-tile bf16 kernel over 6 K) and a ragged, batched one (the general kernel): within 1e-4 of
    the oracle like every fast kernel, and within 2e-6 of the float64 product, i.e. at the level of fp32 accumulation: the
    three cross products that are left out do not show."""
    for (M, N, K, batch) in [(256, 256, 1024, (1, 1, 1)), (200, 136, 1237, (2, 1, 1))]:
        got, want = _run_both(calc, orc, op, M, N, K, abi.FP32, abi.FP32, 0, 0, 0, 0, batch=batch, bcast_b=batch != (1, 1, 1), seed=120 + op,
                              device=True)
        assert rel_frobenius(got, want) <= 1e-4, (M, N, K)
        rng = np.random.default_rng(120 + op)          # the operands _run_both drew
        asz, bsz = _shapes(op, M, N, K)
        nb = int(np.prod(batch))
        a = random_operand(rng, abi.FP32, asz[0] * asz[1] * nb, orc).astype(np.float64).reshape(nb, asz[1], asz[0])
        b = random_operand(rng, abi.FP32, bsz[0] * bsz[1], orc).astype(np.float64).reshape(bsz[1], bsz[0])
        am = a.transpose(0, 2, 1) if op in (abi.OP_ATB, abi.OP_ATBT) else a      # (nb, M, K)
        bm = b.T if op in (abi.OP_ABT, abi.OP_ATBT) else b                        # (K, N)
        exact = (am @ bm).ravel()
        assert rel_frobenius(got, exact) <= 2e-6, (M, N, K)


def test_fp32_three_part_path_keeps_all_24_bits(calc, orc):
    """One-hot operands with full 24-bit significands against powers of two: every product is exact, so the output has to
    reproduce the operand bit for bit at every k position of the six K-blocks."""
    import torch
    M, N, K = 256, 256, 1024
    rng = np.random.default_rng(8)
    a = np.zeros((M, K), np.float32)
    b = np.zeros((K, N), np.float32)
    perm_m = rng.permutation(M)
    vals = (1.0 + rng.integers(1, 1 << 23, K) * 2.0 ** -23).astype(np.float32) * np.where(rng.random(K) < 0.5, -1, 1).astype(np.float32)
    for k in range(K):
        a[perm_m[k % M], k] = vals[k]
        b[k, (k * 11 + 2 + 64 * (k // M)) % N] = 0.5 if k % 2 else 4.0
    want = (a.astype(np.float64) @ b.astype(np.float64)).astype(np.float32)
    out = torch.zeros(M * N, dtype=torch.float32, device="cuda")
    calc.doBatchGemm(MmeSimTensor([N, M], 2, abi.FP32, out), MmeSimTensor([K, M], 2, abi.FP32, torch.from_numpy(a.ravel()).cuda()),
                     MmeSimTensor([N, K], 2, abi.FP32, torch.from_numpy(b.ravel()).cuda()), abi.OP_AB)
    calc.synchronize()
    assert np.array_equal(out.cpu().numpy().reshape(M, N), want)
    # and the other way round: full significands in B
    calc.doBatchGemm(MmeSimTensor([N, M], 2, abi.FP32, out), MmeSimTensor([K, M], 2, abi.FP32, torch.from_numpy((a != 0).astype(np.float32).ravel() * 2).cuda()),
                     MmeSimTensor([N, K], 2, abi.FP32, torch.from_numpy((np.where(b != 0, 1, 0) * vals[:, None]).astype(np.float32).ravel()).cuda()), abi.OP_AB)
    calc.synchronize()
    want2 = ((a != 0).astype(np.float64) * 2) @ (np.where(b != 0, 1, 0) * vals[:, None].astype(np.float64))
    assert np.array_equal(out.cpu().numpy().reshape(M, N).astype(np.float64), want2)


def test_fp32_three_part_path_steps_aside_for_inf_and_nan(calc, orc):
    """inf and NaN among fp32 operands: the contraction runs on the fp32 instantiation instead (decided on the device)."""
    M, N, K = 256, 256, 1024
    rng = np.random.default_rng(11)
    a = rng.standard_normal(M * K).astype(np.float32)
    b = rng.standard_normal(N * K).astype(np.float32)
    a.reshape(M, K)[3, 5], a.reshape(M, K)[7, 9] = np.inf, np.nan
    b.reshape(K, N)[5, 2] = 0.0
    import torch
    out = torch.zeros(M * N, dtype=torch.float32, device="cuda")
    calc.doBatchGemm(MmeSimTensor([N, M], 2, abi.FP32, out), MmeSimTensor([K, M], 2, abi.FP32, torch.from_numpy(a).cuda()),
                     MmeSimTensor([N, K], 2, abi.FP32, torch.from_numpy(b).cuda()), abi.OP_AB)
    calc.synchronize()
    got = out.cpu().numpy().reshape(M, N)
    want = np.zeros(M * N, np.float32)
    assert orc.orc_batch_gemm(A(desc(want, [N, M, 1, 1, 1], abi.FP32)), A(desc(a, [K, M, 1, 1, 1], abi.FP32)), A(desc(b, [N, K, 1, 1, 1], abi.FP32)),
                              abi.OP_AB) == 0
    want = want.reshape(M, N)
    assert np.array_equal(np.isnan(got), np.isnan(want)) and np.isnan(want[3, 2]) and np.isnan(want[7]).all()
    inf = np.isinf(want)
    assert inf.any() and np.array_equal(got[inf], want[inf])
    fin = np.isfinite(want)
    assert rel_frobenius(got[fin], want[fin]) <= 1e-4


@pytest.mark.parametrize("scale_exp", [-115, -126])
def test_fp32_three_part_path_steps_aside_for_tiny_magnitudes(calc, orc, scale_exp):
    """fp32 operands below 2^-100: the low bf16 parts of such values would fall under bf16's range (a = 2^-126 (1 + 2^-8)
    split into bf16 parts loses the 2^-8 entirely), so the contraction must run on the fp32 instantiation.  One operand is
    scaled by 2^scale_exp, the other by 2^100, so that the products are ordinary numbers: against float64, and bit for bit
    on one-hot operands with full 24-bit significands."""
    import torch
    M, N, K = 256, 256, 1024
    rng = np.random.default_rng(21)
    # (random values stay normal fp32 numbers: 2^-115 times a draw; the one-hot values below go down to 2^-126 exactly)
    a = (rng.standard_normal((M, K)).astype(np.float32) * np.float32(2.0 ** max(scale_exp, -115))).astype(np.float32)
    b = (rng.standard_normal((K, N)).astype(np.float32) * np.float32(2.0 ** 100)).astype(np.float32)
    out = torch.zeros(M * N, dtype=torch.float32, device="cuda")

    def run(am, bm):
        calc.doBatchGemm(MmeSimTensor([N, M], 2, abi.FP32, out), MmeSimTensor([K, M], 2, abi.FP32, torch.from_numpy(np.ascontiguousarray(am).ravel()).cuda()),
                         MmeSimTensor([N, K], 2, abi.FP32, torch.from_numpy(np.ascontiguousarray(bm).ravel()).cuda()), abi.OP_AB)
        calc.synchronize()
        return out.cpu().numpy().reshape(M, N).astype(np.float64)

    exact = a.astype(np.float64) @ b.astype(np.float64)
    assert rel_frobenius(run(a, b).ravel(), exact.ravel()) <= 2e-6
    # one-hot: a holds one value per row position k with all 24 significant bits (the advisor's example has 9), b a power of two
    a1 = np.zeros((M, K), np.float32)
    b1 = np.zeros((K, N), np.float32)
    vals = ((1.0 + rng.integers(1, 1 << 23, K) * 2.0 ** -23) * 2.0 ** scale_exp).astype(np.float32)
    vals[0] = np.float32(2.0 ** scale_exp * (1 + 2.0 ** -8))
    for k in range(K):
        a1[(k * 7) % M, k] = vals[k]
        b1[k, (k * 11 + 2 + 64 * (k // M)) % N] = np.float32(2.0 ** 110)
    want = a1.astype(np.float64) @ b1.astype(np.float64)
    assert np.array_equal(run(a1, b1), want)
    # and a later call with ordinary operands takes the split path again (the flag holds the earlier call's epoch)
    a2, b2 = rng.standard_normal((M, K)).astype(np.float32), rng.standard_normal((K, N)).astype(np.float32)
    assert rel_frobenius(run(a2, b2).ravel(), (a2.astype(np.float64) @ b2.astype(np.float64)).ravel()) <= 2e-6


PERSISTENT = [  # op, dtA, bA, dtB, bB, out_dt, out_bias, M, N, K, batch, rows per reference launch
    (abi.OP_AB, abi.FP8_143, 7, abi.FP8_143, 7, abi.BF16, 0, 4096, 8192, 384, 1, 1024),      # 16 x 32 tiles: 8 x 4 blocks per XCD
    (abi.OP_ABT, abi.FP8_152, 15, abi.FP8_143, 11, abi.FP8_143, 7, 2560, 13312, 512, 1, 1280),  # 10 x 52 tiles: row-major walk
    (abi.OP_AB, abi.FP8_143, 7, abi.FP8_152, 15, abi.FP8_152, 15, 1280, 13312, 384, 2, 1280),   # two batch elements, B broadcast
    (abi.OP_AB, abi.BF16, 0, abi.BF16, 0, abi.BF16, 0, 4096, 8192, 192, 1, 1024),               # bf16 operands
    (abi.OP_ABT, abi.BF16, 0, abi.BF16, 0, abi.FP8_143, 7, 2560, 13312, 256, 1, 1280),
]


@pytest.mark.parametrize("op,dtA,bA,dtB,bB,out_dt,out_bias,M,N,K,batch,rows", PERSISTENT)
def test_persistent_walk_equals_tile_by_tile_launches(calc, orc, op, dtA, bA, dtB, bB, out_dt, out_bias, M, N, K, batch, rows):
    """Problems with at least 512 tiles take the kernel whose workgroups walk over tiles (next tile's first stages requested
    before the finished tile's epilogue).  The same problem launched slab by slab (fewer than 512 tiles per launch: one
    workgroup per tile, the kernel the other tests hold against the oracle) must give the same output codes."""
    import torch
    rng = np.random.default_rng(77)
    a = random_operand(rng, dtA, M * K * batch, orc, bA)
    b = random_operand(rng, dtB, N * K, orc, bB, scale=0.05)
    col = torch.from_numpy(rng.integers(-3, 4, N).astype(np.int32)).cuda()
    ta = torch.from_numpy(a.view(np.int16) if dtA == abi.BF16 else a).cuda()
    tb = torch.from_numpy(b.view(np.int16) if dtB == abi.BF16 else b).cuda()
    td = torch.int16 if out_dt == abi.BF16 else torch.uint8
    bsz = [K, N] if op == abi.OP_ABT else [N, K]
    W = MmeSimTensor(bsz + ([1] if batch > 1 else []), 3 if batch > 1 else 2, dtB, tb, bB)
    epi = Epilogue(scale_exp=-4, col_scale_exp=col, clipFp=True)

    whole = torch.zeros(M * N * batch, dtype=td, device="cuda")
    X = MmeSimTensor([K, M] + ([batch] if batch > 1 else []), 3 if batch > 1 else 2, dtA, ta, bA)
    calc.doBatchGemm(MmeSimTensor([N, M] + ([batch] if batch > 1 else []), 3 if batch > 1 else 2, out_dt, whole, out_bias), X, W, op, epilogue=epi)

    W2 = MmeSimTensor(bsz, 2, dtB, tb, bB)
    parts = torch.zeros(M * N * batch, dtype=td, device="cuda")
    assert (rows // 256) * (N // 256) < 512 and (M * batch) % rows == 0
    for r0 in range(0, M * batch, rows):
        Xs = MmeSimTensor([K, rows], 2, dtA, ta[r0 * K:(r0 + rows) * K], bA)
        calc.doBatchGemm(MmeSimTensor([N, rows], 2, out_dt, parts[r0 * N:(r0 + rows) * N], out_bias), Xs, W2, op, epilogue=epi)
    calc.synchronize()
    got, want = whole.cpu().numpy(), parts.cpu().numpy()
    assert np.count_nonzero(want) > want.size // 2
    assert np.array_equal(got, want)
