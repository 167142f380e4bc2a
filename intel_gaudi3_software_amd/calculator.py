"""Python mirror of the reference calculator's host API over the C ABI (``include/mme_hip.h``).

``HipCalculator`` has the method names, argument order and error behaviour of ``CPUCalculator``
(mme/mme_reference/mme_reference.h:108-191); ``MmeSimTensor`` has the constructor arguments of the reference class of
that name (mme/mme_reference/sim_tensor.h:13-19).  It exists so that tests and the benchmark can drive the library the
way the reference's own tests drive the calculator (mme/tests/unit_tests/mme_unit_test.cpp:67-172); the C++ form of the
same surface is ``include/mme_hip_calculator.h``.

A tensor wraps either host memory (a numpy array) or device memory (a torch tensor on ``cuda``); the calculator picks
the host-pointer or the ``_dev`` entry point accordingly.  There is no CPU fallback.
"""
import ctypes as C

import numpy as np

from . import abi
from .abi import (BF16, FP8_143, FP8_152, FP32, FULL_INF_NAN, OP_AB, OP_ABT, OP_ATB, OP_ATBT, OP_DEDW, OP_DEDX, OP_FWD,
                  RM_NEAREST_EVEN)


class MMEStackException(RuntimeError):
    """What MME_ASSERT throws in the reference's release builds (mme/include/mme_assert.h:19-58)."""

    def __init__(self, message, status=abi.EINVAL):
        super().__init__(message)
        self.status = status


class MmeSimTensor:
    """Descriptor + storage.  ``sizes[0]`` is the contiguous dimension (sim_tensor_base.h:52-54).

    ``data`` may be a numpy array (host), a torch tensor (host or device) or None (zero-filled host storage is
    allocated, like sim_tensor_base.cpp:401-405).  The buffer is viewed flat; ``strides`` are in elements.
    """

    def __init__(self, sizes, dim, dtype, data=None, fpBias=0, infNanMode=FULL_INF_NAN, strides=None):
        self.sizes = list(sizes) + [1] * (abi.MAX_TENSOR_DIMS - len(sizes))
        self.dim = dim
        self.dtype = dtype
        self.fpBias = fpBias
        self.infNanMode = infNanMode
        if strides is None:
            strides, acc = [], 1
            for s in self.sizes:
                strides.append(acc)
                acc *= s
        else:
            strides = list(strides)
            while len(strides) < abi.MAX_TENSOR_DIMS:
                strides.append(strides[-1] * self.sizes[len(strides) - 1])
        self.strides = strides
        span = max(st * sz for st, sz in zip(self.strides, self.sizes))
        self.is_device = False
        if data is None:
            data = np.zeros(max(span, 1), dtype=abi.DTYPE_NUMPY[dtype])
        if isinstance(data, np.ndarray):
            if data.dtype.itemsize != abi.DTYPE_SIZE[dtype]:
                raise ValueError("array item size does not match the tensor type")
            if data.size < span:
                raise ValueError("buffer too small for sizes/strides")
            if not data.flags["C_CONTIGUOUS"]:
                raise ValueError("buffer must be contiguous")
            self._keep = data
            self._ptr = data.ctypes.data
        else:  # torch tensor
            if data.element_size() != abi.DTYPE_SIZE[dtype]:
                raise ValueError("tensor item size does not match the tensor type")
            if data.numel() < span:
                raise ValueError("buffer too small for sizes/strides")
            if not data.is_contiguous():
                raise ValueError("buffer must be contiguous")
            self._keep = data
            self._ptr = data.data_ptr()
            self.is_device = data.is_cuda
        self.desc = abi.make_tensor(self._ptr, self.sizes, dtype, fpBias, infNanMode, self.strides, dim)

    # accessors named after the reference's (sim_tensor_base.h:60-90)
    def data(self):
        return self._keep

    def getDim(self):
        return self.dim

    def getSizes(self):
        return list(self.sizes)

    def getStrides(self):
        return list(self.strides)

    def getSizeInElements(self):
        n = 1
        for s in self.sizes:
            n *= s
        return n

    def getElementType(self):
        return self.dtype

    def getFpBias(self):
        return self.fpBias

    def getInfNanMode(self):
        return self.infNanMode


class ConvolutionParams:
    """mme/mme_reference/convolution_params.h:7-29: dim, padding / convStride / dilation indexed W, H, D(, batch)."""

    def __init__(self, dim=3, padding=(0, 0, 0, 0), convStride=(1, 1, 1, 1), dilation=(1, 1, 1, 1), relu=False):
        self.dim = dim
        self.padding = list(padding)
        self.convStride = list(convStride)
        self.dilation = list(dilation)
        self.relu = relu

    def pod(self):
        return abi.make_conv_params(self.dim, self.padding, self.convStride, self.dilation, self.relu)


class Epilogue:
    """Fused descale + relu + cast behind a contraction (``mme_hip_epilogue``)."""

    def __init__(self, scale_exp=0, col_scale_exp=None, relu=False, rm=RM_NEAREST_EVEN, clipFp=False, clipInfIn=False,
                 flushDenorms=False):
        self._col = col_scale_exp  # int32 device tensor or None
        e = abi.Epilogue()
        e.scale_exp = scale_exp
        e.col_scale_exp = col_scale_exp.data_ptr() if col_scale_exp is not None else None
        e.relu = int(relu)
        e.rounding_mode = rm
        e.clip_fp = int(clipFp)
        e.clip_inf_in = int(clipInfIn)
        e.flush_denorms = int(flushDenorms)
        self.pod = e


class HipCalculator:
    """``CPUCalculator`` (mme/mme_reference/mme_reference.h:108-191) on one MI355X."""

    def __init__(self, chip=abi.CHIP_GAUDI3, max_tensor_dims=abi.MAX_TENSOR_DIMS, max_conv_dims=abi.MAX_CONV_DIMS, seed=0,
                 lfsrNumRegs=256, lfsr=None, polynomial=0):
        self._lib = abi.load_library()
        self._h = C.c_void_p()
        lf = None
        if lfsr is not None:
            self._lfsr_in = np.ascontiguousarray(lfsr, dtype=np.uint32)
            lf = self._lfsr_in.ctypes.data
        rc = self._lib.mme_hip_create(C.byref(self._h), chip, max_tensor_dims, max_conv_dims, seed, lfsrNumRegs, lf, polynomial)
        if rc != 0:
            raise MMEStackException(self._lib.mme_hip_last_error(None).decode(), rc)
        self._caller_stream = False
        self._in_flight = []   # device operands of calls since the last synchronize()

    def close(self):
        if getattr(self, "_h", None) is not None and self._h.value:
            self._lib.mme_hip_destroy(self._h)   # (waits for the stream)
            self._h = C.c_void_p()
            self._in_flight = []

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def _check(self, rc):
        if rc != 0:
            raise MMEStackException(self._lib.mme_hip_last_error(self._h).decode(), rc)

    # ---- the reference's methods ------------------------------------------------------------------------------------
    def limitNumOfThreads(self, numOfThreads):
        self._check(self._lib.mme_hip_limit_num_of_threads(self._h, numOfThreads))

    def doBatchGemm(self, outputTensor, xTensor, wTensor, op, rm=RM_NEAREST_EVEN, clipFp=False, clipFpInfIn=False,
                    epilogue=None):
        dev = self._placement(outputTensor, xTensor, wTensor)
        if dev:
            self._check(self._lib.mme_hip_set_operand_clip(self._h, int(clipFp), int(clipFpInfIn)))
            self._check(self._lib.mme_hip_batch_gemm_dev(self._h, outputTensor.desc, xTensor.desc, wTensor.desc, op,
                                                         epilogue.pod if epilogue else None))
        else:
            if epilogue is not None:
                raise MMEStackException("the fused epilogue needs device tensors", abi.EINVAL)
            self._check(self._lib.mme_hip_batch_gemm(self._h, outputTensor.desc, xTensor.desc, wTensor.desc, op, rm,
                                                     int(clipFp), int(clipFpInfIn)))

    def doConvolution(self, outputTensor, xTensor, wTensor, yTensor, params, op, rm=RM_NEAREST_EVEN, clipFp=False,
                      clipFpInfIn=False, epilogue=None):
        dev = self._placement(outputTensor, xTensor, wTensor, yTensor)
        pod = params.pod()
        if dev:
            self._check(self._lib.mme_hip_set_operand_clip(self._h, int(clipFp), int(clipFpInfIn)))
            self._check(self._lib.mme_hip_convolution_dev(self._h, outputTensor.desc, xTensor.desc, wTensor.desc, yTensor.desc,
                                                          pod, op, epilogue.pod if epilogue else None))
        else:
            if epilogue is not None:
                raise MMEStackException("the fused epilogue needs device tensors", abi.EINVAL)
            self._check(self._lib.mme_hip_convolution(self._h, outputTensor.desc, xTensor.desc, wTensor.desc, yTensor.desc, pod,
                                                      op, rm, int(clipFp), int(clipFpInfIn)))

    def doActivation(self, output, acc, res=None, bias=None, relu=False, rm=RM_NEAREST_EVEN, actParams=None, clipFp=False,
                     clipInfIn=False, flushDenorms=False, stochasticFTZfp8=False):
        if actParams is not None:
            raise MMEStackException("activationGemmlowp (integer requantisation) is not built in this library",
                                    abi.EUNSUPPORTED)
        dev = self._placement(output, acc)
        fn = self._lib.mme_hip_activation_dev if dev else self._lib.mme_hip_activation
        self._check(fn(self._h, output.desc, acc.desc, int(relu), rm, int(clipFp), int(clipInfIn), int(flushDenorms),
                       int(stochasticFTZfp8)))

    def doMemoryWrite(self, memory, mmeOut, reductionOp=abi.REDUCTION_NONE, reductionRm=0, clipFp=False):
        dev = self._placement(memory, mmeOut)
        fn = self._lib.mme_hip_memory_write_dev if dev else self._lib.mme_hip_memory_write
        self._check(fn(self._h, memory.desc, mmeOut.desc, reductionOp, reductionRm, int(clipFp)))

    # ---- extensions of the GPU path ------------------------------------------------------------------------------------
    def synchronize(self):
        self._check(self._lib.mme_hip_synchronize(self._h))
        self._in_flight.clear()

    def stream(self):
        return self._lib.mme_hip_stream(self._h)

    def setStream(self, hip_stream):
        """Enqueue on a caller-owned stream (0 / None: back to the calculator's own).  With a caller-owned stream the
        ordering against the producers of the operands is the caller's business; on its own stream the calculator waits,
        on the device, for what torch's current stream has enqueued so far before every call on torch tensors."""
        self._check(self._lib.mme_hip_set_stream(self._h, hip_stream))
        self._caller_stream = bool(hip_stream)

    def _after_torch(self, *device_tensors):
        # the calculator's own stream does not synchronise with any other: make it wait (on the device) for the fills and
        # copies that produced the operands on torch's current stream, and keep the operands referenced until the next
        # synchronize(), so that a temporary passed inline is not released to torch's allocator (and handed to the next
        # allocation) while a kernel still reads it.  Results may be consumed on torch's stream after synchronize().
        if self._caller_stream:
            return
        import torch
        ev = torch.cuda.Event()
        ev.record()
        torch.cuda.ExternalStream(self.stream()).wait_event(ev)
        self._in_flight.extend(t for t in device_tensors if t is not None and getattr(t, "is_cuda", False))
        if len(self._in_flight) > 512:
            self.synchronize()

    def setWaitLimit(self, polls):
        """Bound on the polls of a kernel's internal waits (mme_hip_set_wait_limit); a wait that runs out is reported by the
        next synchronize()."""
        self._check(self._lib.mme_hip_set_wait_limit(self._h, polls))

    def clockProbe(self, enable=True):
        """Diagnostics (mme_hip_clock_probe): the large-tile kernels note clock counters per workgroup while this is on."""
        self._check(self._lib.mme_hip_clock_probe(self._h, int(bool(enable))))

    def readClockProbe(self):
        """Synchronises and returns {shader_mhz, workgroup_us_mean, workgroup_us_max, workgroups} over the workgroups that ran
        since the last read (mme_hip_clock_probe_read)."""
        import ctypes as C
        mhz, mean, worst, n = C.c_double(), C.c_double(), C.c_double(), C.c_int()
        self._check(self._lib.mme_hip_clock_probe_read(self._h, C.byref(mhz), C.byref(mean), C.byref(worst), C.byref(n)))
        self._in_flight.clear()
        return {"shader_mhz": mhz.value, "workgroup_us_mean": mean.value, "workgroup_us_max": worst.value, "workgroups": n.value}

    def lastContractionForm(self):
        """Which kernel form the latest doBatchGemm / doConvolution launched (mme_hip_last_contraction_form):
        {large_tile, tile_rows, split_k, wavefronts}."""
        import ctypes as C
        v = [C.c_int() for _ in range(4)]
        self._check(self._lib.mme_hip_last_contraction_form(self._h, *[C.byref(x) for x in v]))
        return {"large_tile": bool(v[0].value), "tile_rows": v[1].value, "split_k": v[2].value, "wavefronts": v[3].value}

    def matrixCoreRate(self, dtype, random_operands, iters=4096, launches=10):
        """(TFLOP/s, shader clock in MHz) of back-to-back matrix instructions with operands in registers
        (mme_hip_matrix_core_rate): what the matrix cores sustain on this device and this kind of data."""
        import ctypes as C
        tf, mhz = C.c_double(), C.c_double()
        self._check(self._lib.mme_hip_matrix_core_rate(self._h, dtype, int(bool(random_operands)), iters, launches, C.byref(tf), C.byref(mhz)))
        return tf.value, mhz.value

    def setFp8SpecialsPolicy(self, policy):
        self._check(self._lib.mme_hip_set_fp8_specials_policy(self._h, policy))

    def castFromFp32(self, out, out_dtype, src, n, fpBias=0, infNanMode=FULL_INF_NAN, scale_exp=0, col_scale_exp=None,
                     n_cols=0, relu=False, rm=RM_NEAREST_EVEN, clipFp=False, clipInfIn=False, flushDenorms=False):
        """Flat quantise / cast on device buffers (torch tensors)."""
        self._after_torch(out, src, col_scale_exp)
        self._check(self._lib.mme_hip_cast_from_fp32_dev(
            self._h, out.data_ptr(), out_dtype, fpBias, infNanMode, src.data_ptr(), n, scale_exp,
            col_scale_exp.data_ptr() if col_scale_exp is not None else None, n_cols, int(relu), rm, int(clipFp), int(clipInfIn),
            int(flushDenorms)))

    def castToFp32(self, out, src, in_dtype, n, fpBias=0, infNanMode=FULL_INF_NAN, scale_exp=0, col_scale_exp=None, n_cols=0):
        """Flat dequantise on device buffers (torch tensors)."""
        self._after_torch(out, src, col_scale_exp)
        self._check(self._lib.mme_hip_cast_to_fp32_dev(
            self._h, out.data_ptr(), src.data_ptr(), in_dtype, fpBias, infNanMode, n, scale_exp,
            col_scale_exp.data_ptr() if col_scale_exp is not None else None, n_cols))

    def absmax(self, out, src, n):
        self._after_torch(out, src)
        self._check(self._lib.mme_hip_absmax_dev(self._h, out.data_ptr(), src.data_ptr(), n))

    def _placement(self, *tensors):
        dev = [t.is_device for t in tensors]
        if any(dev) and not all(dev):
            raise MMEStackException("tensors of one call must all be host or all be device resident", abi.EINVAL)
        if all(dev):
            self._after_torch(*[t.data() for t in tensors])
        return all(dev)
