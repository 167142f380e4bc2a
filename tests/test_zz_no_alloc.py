"""The entry point that allocates nothing, mme_hip_batch_gemm_dev_noalloc, through the C ABI: bit-identical outputs to
mme_hip_batch_gemm_dev (the same kernels, the work spaces in the device's static scratch array instead of buffers the
handle allocates) on calls in a row, the later ones with smaller inputs; no change in free device memory across the calls;
a clear error for a problem whose work space exceeds the array."""
import ctypes as C

import numpy as np
import pytest

from intel_gaudi3_software_amd import abi

pytestmark = pytest.mark.gpu


def _handle(lib):
    h = C.c_void_p()
    assert lib.mme_hip_create(C.byref(h), abi.CHIP_GAUDI3, 5, 4, 0, 256, None, 0) == 0, lib.mme_hip_last_error(None)
    return h


def _bf16(x):
    u = np.asarray(x, np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def _run(lib, h, fn, a, b, out, sizes_a, sizes_b, sizes_o, dt, bias, mode, out_dt, op, epi):
    ta = abi.make_tensor(a.data_ptr(), sizes_a, dt, bias, mode)
    tb = abi.make_tensor(b.data_ptr(), sizes_b, dt, bias, mode)
    to = abi.make_tensor(out.data_ptr(), sizes_o, out_dt)
    rc = fn(h, C.byref(to), C.byref(ta), C.byref(tb), op, C.byref(epi) if epi is not None else None)
    return rc


def test_no_alloc_entry_point_equals_the_allocating_one():
    import torch
    lib = abi.load_library()
    h = _handle(lib)
    rng = np.random.default_rng(41)
    try:
        # (dtype, bias, mode, M, N, K, output type): split-k partial sums (one tile, long reduction), then smaller inputs,
        # then fp8 operands that hold an inf code (flag cell + decoded copies from the scratch), then a smaller clean fp8 call
        cases = [("bf16", abi.BF16, 0, 0, 256, 256, 8192, abi.FP32),
                 ("bf16 smaller", abi.BF16, 0, 0, 128, 256, 4096, abi.FP32),
                 ("fp8 with inf", abi.FP8_143, 7, 0, 512, 256, 1024, abi.FP32),
                 ("fp8 smaller, clean, fused", abi.FP8_143, 7, 0, 256, 256, 512, abi.BF16),
                 ("fp32 (three bf16 parts)", abi.FP32, 0, 0, 256, 256, 1024, abi.FP32),
                 ("ragged bf16", abi.BF16, 0, 0, 70, 52, 3000, abi.FP32)]
        for i, (name, dt, bias, mode, M, N, K, out_dt) in enumerate(cases):
            if dt == abi.BF16:
                a = torch.from_numpy(_bf16(rng.standard_normal(M * K)).view(np.int16)).cuda()
                b = torch.from_numpy(_bf16(rng.standard_normal(K * N)).view(np.int16)).cuda()
            elif dt == abi.FP32:
                a = torch.from_numpy(rng.standard_normal(M * K).astype(np.float32)).cuda()
                b = torch.from_numpy(rng.standard_normal(K * N).astype(np.float32)).cuda()
            else:
                ca = rng.integers(0, 0x60, M * K).astype(np.uint8) | (rng.integers(0, 2, M * K).astype(np.uint8) << 7)
                cb = rng.integers(0, 0x60, K * N).astype(np.uint8) | (rng.integers(0, 2, K * N).astype(np.uint8) << 7)
                if "inf" in name:
                    ca[37 * K + 700] = 0x78
                a, b = torch.from_numpy(ca).cuda(), torch.from_numpy(cb).cuda()
            tdt = torch.float32 if out_dt == abi.FP32 else torch.int16
            o1 = torch.full((M * N,), 7, dtype=tdt, device="cuda")
            o2 = torch.full((M * N,), 9, dtype=tdt, device="cuda")
            epi = None
            if out_dt != abi.FP32:
                epi = abi.Epilogue()
                epi.scale_exp = -3
                epi.clip_fp = 1
            torch.cuda.synchronize()
            print("no-alloc case:", name, M, N, K, flush=True)
            assert _run(lib, h, lib.mme_hip_batch_gemm_dev, a, b, o1, [K, M], [N, K], [N, M], dt, bias, mode, out_dt, abi.OP_AB, epi) == 0, lib.mme_hip_last_error(h)
            assert lib.mme_hip_synchronize(h) == 0
            assert _run(lib, h, lib.mme_hip_batch_gemm_dev_noalloc, a, b, o2, [K, M], [N, K], [N, M], dt, bias, mode, out_dt, abi.OP_AB, epi) == 0, lib.mme_hip_last_error(h)
            assert lib.mme_hip_synchronize(h) == 0
            r1, r2 = o1.cpu().numpy(), o2.cpu().numpy()
            assert np.array_equal(r1.view(np.uint8), r2.view(np.uint8)), name
            assert np.any(r1 != 7)
            if "inf" in name:
                # (inf times a zero of B is NaN)
                assert not np.isfinite(r1.reshape(M, N)[37]).any() and np.isfinite(np.delete(r1.reshape(M, N), 37, axis=0)).all()
        # the second call of a pair never allocates: across a few more of them the free device memory does not move
        a = torch.from_numpy(_bf16(rng.standard_normal(128 * 4096)).view(np.int16)).cuda()
        b = torch.from_numpy(_bf16(rng.standard_normal(4096 * 256)).view(np.int16)).cuda()
        o = torch.zeros(128 * 256, dtype=torch.float32, device="cuda")
        torch.cuda.synchronize()
        free0 = torch.cuda.mem_get_info()[0]
        for _ in range(5):
            assert _run(lib, h, lib.mme_hip_batch_gemm_dev_noalloc, a, b, o, [4096, 128], [256, 4096], [256, 128], abi.BF16, 0, 0, abi.FP32, abi.OP_AB, None) == 0
        assert lib.mme_hip_synchronize(h) == 0
        assert torch.cuda.mem_get_info()[0] == free0
        # too large for the array: 4096^3 fp8 in full inf/NaN mode needs 64 MiB of decoded copies for its fall-back
        n = 4096
        big_a = torch.zeros(n * n, dtype=torch.uint8, device="cuda")
        big_o = torch.zeros(n * n, dtype=torch.float32, device="cuda")
        rc = _run(lib, h, lib.mme_hip_batch_gemm_dev_noalloc, big_a, big_a, big_o, [n, n], [n, n], [n, n], abi.FP8_143, 7, 0, abi.FP32, abi.OP_AB, None)
        assert rc == abi.ENOMEM and b"static scratch" in lib.mme_hip_last_error(h)
        assert lib.mme_hip_synchronize(h) == 0
        # ... and with the caller's word that the operands hold no such codes it needs no work space at all
        assert lib.mme_hip_set_fp8_specials_policy(h, abi.FP8_SPECIALS_ASSUME_NONE) == 0
        assert _run(lib, h, lib.mme_hip_batch_gemm_dev_noalloc, big_a, big_a, big_o, [n, n], [n, n], [n, n], abi.FP8_143, 7, 0, abi.FP32, abi.OP_AB, None) == 0
        assert lib.mme_hip_synchronize(h) == 0
    finally:
        lib.mme_hip_destroy(h)


def test_no_alloc_entry_point_first_on_a_fresh_handle():
    """A handle whose very first calls go through the entry point that allocates nothing: split-k bf16, fp8 operands with an
    inf code (flag cell and decoded copies), fp32 operands (three bf16 parts) and a fused epilogue with stochastic rounding
    (the LFSR jump table must exist since mme_hip_create).  The free device memory does not move across those calls, and
    the outputs equal those of a second handle that takes the allocating entry point (which also runs first, so that the
    code objects are loaded and torch's allocator holds its blocks before free memory is read)."""
    import torch
    lib = abi.load_library()
    rng = np.random.default_rng(43)

    def operands(dt, M, N, K):
        if dt == abi.BF16:
            return (torch.from_numpy(_bf16(rng.standard_normal(M * K)).view(np.int16)).cuda(), torch.from_numpy(_bf16(rng.standard_normal(K * N)).view(np.int16)).cuda())
        if dt == abi.FP32:
            return (torch.from_numpy(rng.standard_normal(M * K).astype(np.float32)).cuda(), torch.from_numpy(rng.standard_normal(K * N).astype(np.float32)).cuda())
        ca = rng.integers(0, 0x60, M * K).astype(np.uint8) | (rng.integers(0, 2, M * K).astype(np.uint8) << 7)
        cb = rng.integers(0, 0x60, K * N).astype(np.uint8) | (rng.integers(0, 2, K * N).astype(np.uint8) << 7)
        return torch.from_numpy(ca).cuda(), torch.from_numpy(cb).cuda()

    # (name, dtype, bias, M, N, K, output type, rounding mode of the fused epilogue or None, code to plant in A)
    cases = [("bf16 split-k", abi.BF16, 0, 256, 256, 8192, abi.FP32, None, None),
             ("fp8 with inf", abi.FP8_143, 7, 512, 256, 1024, abi.FP32, None, 0x78),
             ("fp32 three parts", abi.FP32, 0, 256, 256, 1024, abi.FP32, None, None),
             ("fp8 stochastic epilogue", abi.FP8_143, 7, 256, 256, 512, abi.BF16, 4, None)]
    data = []
    for name, dt, bias, M, N, K, out_dt, rm, plant in cases:
        a, b = operands(dt, M, N, K)
        if plant is not None:
            a[11 * K + 5] = plant
        tdt = torch.float32 if out_dt == abi.FP32 else torch.int16
        epi = None
        if rm is not None:
            epi = abi.Epilogue()
            epi.scale_exp = -3
            epi.rounding_mode = rm
            epi.clip_fp = 1
        data.append((name, dt, bias, M, N, K, out_dt, epi, a, b, torch.full((M * N,), 7, dtype=tdt, device="cuda"), torch.full((M * N,), 9, dtype=tdt, device="cuda")))
    h_alloc = _handle(lib)
    try:
        for name, dt, bias, M, N, K, out_dt, epi, a, b, o1, o2 in data:
            assert _run(lib, h_alloc, lib.mme_hip_batch_gemm_dev, a, b, o1, [K, M], [N, K], [N, M], dt, bias, 0, out_dt, abi.OP_AB, epi) == 0, lib.mme_hip_last_error(h_alloc)
        assert lib.mme_hip_synchronize(h_alloc) == 0
        h = _handle(lib)
        try:
            torch.cuda.synchronize()
            free0 = torch.cuda.mem_get_info()[0]
            for name, dt, bias, M, N, K, out_dt, epi, a, b, o1, o2 in data:
                print("no-alloc first on a fresh handle:", name, flush=True)
                assert _run(lib, h, lib.mme_hip_batch_gemm_dev_noalloc, a, b, o2, [K, M], [N, K], [N, M], dt, bias, 0, out_dt, abi.OP_AB, epi) == 0, lib.mme_hip_last_error(h)
                assert lib.mme_hip_synchronize(h) == 0
            assert torch.cuda.mem_get_info()[0] == free0
            for name, dt, bias, M, N, K, out_dt, epi, a, b, o1, o2 in data:
                r1, r2 = o1.cpu().numpy(), o2.cpu().numpy()
                assert np.array_equal(r1.view(np.uint8), r2.view(np.uint8)), name
                assert np.any(r1 != 7), name
        finally:
            lib.mme_hip_destroy(h)
    finally:
        lib.mme_hip_destroy(h_alloc)
