import numpy as np
import pytest

from intel_gaudi3_software_amd import MmeSimTensor, abi
from helpers import A, desc, rel_frobenius

pytestmark = pytest.mark.gpu


def test_fp8_one_round_gemm_recorded_into_a_graph_settles_special_codes_on_every_replay(orc):
    """A one-round fp8 GEMM (3072 x 4096 outputs, K = 3072) enqueued while its stream records a graph.  Called directly, such a
    launch settles special codes through words that the host hands out per launch; a recorded launch keeps the words of the
    moment it was recorded, so the library must give it the form that is safe to run again and again.  Replays with clean
    operands, with a special code in A, clean again, with one in B, clean again, direct calls in between: every replay
    against the direct call on the same operands and, for the rows that the codes touch, against the oracle."""
    import torch
    from intel_gaudi3_software_amd import HipCalculator
    M, N, K = 3072, 4096, 3072
    rng = np.random.default_rng(77)
    a0 = (rng.integers(0, 0x58, M * K).astype(np.uint8) | (rng.integers(0, 2, M * K).astype(np.uint8) << 7)).reshape(M, K)
    b0 = (rng.integers(0, 0x58, K * N).astype(np.uint8) | (rng.integers(0, 2, K * N).astype(np.uint8) << 7)).reshape(K, N)
    c = HipCalculator()
    try:
        ta, tb = torch.from_numpy(a0.ravel().copy()).cuda(), torch.from_numpy(b0.ravel().copy()).cuda()
        out = torch.zeros(M * N, dtype=torch.float32, device="cuda")
        X, Wt, Y = MmeSimTensor([K, M], 2, abi.FP8_143, ta, 7), MmeSimTensor([N, K], 2, abi.FP8_143, tb, 7), MmeSimTensor([N, M], 2, abi.FP32, out)
        # work spaces only grow and a recording stream cannot allocate: a direct call over two batch elements of the same
        # operands (384 tiles, more than one round: the form that a recorded call takes) sizes them beforehand
        ta2, out2 = torch.cat([ta, ta]), torch.zeros(2 * M * N, dtype=torch.float32, device="cuda")
        c.doBatchGemm(MmeSimTensor([N, M, 2, 1, 1], 5, abi.FP32, out2), MmeSimTensor([K, M, 2, 1, 1], 5, abi.FP8_143, ta2, 7),
                      MmeSimTensor([N, K, 1, 1, 1], 5, abi.FP8_143, tb, 7), abi.OP_AB)
        c.synchronize()
        del ta2, out2
        side = torch.cuda.Stream()
        torch.cuda.synchronize()
        c.setStream(side.cuda_stream)

        def direct():
            out.zero_()
            torch.cuda.synchronize()
            c.doBatchGemm(Y, X, Wt, abi.OP_AB)
            form = c.lastContractionForm()
            assert form["large_tile"] and form["wavefronts"] == 4 and form["split_k"] == 1, form
            c.synchronize()
            return out.cpu().numpy().reshape(M, N)

        clean = direct()
        assert np.isfinite(clean).all()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            c.doBatchGemm(Y, X, Wt, abi.OP_AB)
        torch.cuda.synchronize()

        def replayed():
            out.zero_()
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            return out.cpu().numpy().reshape(M, N)

        def oracle_rows(a, b, rows):
            want = np.zeros(rows.size * N, np.float32)
            slab = np.ascontiguousarray(a[rows].ravel())
            assert orc.orc_batch_gemm(A(desc(want, [N, rows.size], abi.FP32)), A(desc(slab, [K, rows.size], abi.FP8_143, 7)),
                                      A(desc(b.ravel(), [N, K], abi.FP8_143, 7)), abi.OP_AB) == 0
            return want.reshape(rows.size, N)

        states = [("clean", None), ("a", (2 * 256 + 131, 64 * 20 + 7, 0x78)), ("clean", None), ("b", (64 * 31 + 60, 9 * 256 + 3, 0x7D)), ("clean", None)]
        for step, (which, place) in enumerate(states):
            a, b = a0.copy(), b0.copy()
            if which == "a":
                a[place[0], place[1]] = place[2]   # +inf in row 643
            elif which == "b":
                b[place[0], place[1]] = place[2]   # NaN in column 2307
            ta.copy_(torch.from_numpy(a.ravel()))
            tb.copy_(torch.from_numpy(b.ravel()))
            torch.cuda.synchronize()
            got = replayed()
            want = direct()
            assert np.array_equal(np.isnan(got), np.isnan(want)), (step, which)
            inf = np.isinf(want)
            assert np.array_equal(got[inf], want[inf]), (step, which)
            fin = np.isfinite(want)
            assert rel_frobenius(got[fin], want[fin]) <= 1e-4, (step, which)
            if which == "clean":
                # (bit-equal to the first result only until a replay has met a special code: from then on the replays may
                # keep running the exactly decoded form, whose sums are taken in another order)
                assert np.isfinite(got).all() and (np.array_equal(got, clean) if step == 0 else rel_frobenius(got, clean) <= 1e-4), step
            else:
                assert not np.isfinite(got).all(), (step, which)
                rows = np.array([0, 643, 1500, M - 1])
                ref = oracle_rows(a, b, rows)
                g = got[rows]
                assert np.array_equal(np.isnan(g), np.isnan(ref)) and np.array_equal(np.isinf(g), np.isinf(ref)), (step, which)
                f = np.isfinite(ref)
                assert np.array_equal(g[~f & ~np.isnan(ref)], ref[~f & ~np.isnan(ref)]) and rel_frobenius(g[f], ref[f]) <= 1e-4, (step, which)
        # a larger direct call on the same handle outgrows the work space that the recorded fall-back launches point into (the
        # decoded copies of three batch elements of A): the handle has seen a recording stream, so it keeps the old block,
        # and a replay that meets a special code still computes the right thing
        ta3, out3 = torch.cat([ta, ta, ta]), torch.zeros(3 * M * N, dtype=torch.float32, device="cuda")
        c.doBatchGemm(MmeSimTensor([N, M, 3, 1, 1], 5, abi.FP32, out3), MmeSimTensor([K, M, 3, 1, 1], 5, abi.FP8_143, ta3, 7),
                      MmeSimTensor([N, K, 1, 1, 1], 5, abi.FP8_143, tb, 7), abi.OP_AB)
        c.synchronize()
        del ta3, out3
        spare = [torch.full((1 << 22,), 1.5, dtype=torch.float32, device="cuda") for _ in range(8)]  # would land in a freed block
        a = a0.copy()
        a[5, 9] = 0x78
        ta.copy_(torch.from_numpy(a.ravel()))
        tb.copy_(torch.from_numpy(b0.ravel()))
        torch.cuda.synchronize()
        got, want = replayed(), direct()
        assert np.array_equal(np.isnan(got), np.isnan(want)) and np.array_equal(np.isinf(got), np.isinf(want))
        fin = np.isfinite(want)
        assert not fin.all() and rel_frobenius(got[fin], want[fin]) <= 1e-4
        assert all(float(t.min()) == 1.5 and float(t.max()) == 1.5 for t in spare)
        del graph, spare
    finally:
        c.setStream(None)
        c.close()
