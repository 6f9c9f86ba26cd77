"""Host-side mirror of the reference's GPUWrapper / GPUTensor<float> for the Dot path.

Names, argument meaning and error behaviour follow the C# classes so the parity
tests read like the reference's own (Tests/GPU/TestGpuTensor.cs,
Tests/TestParallelRunCpuVersusGpu.cs):

* ``GPUWrapper``  - per-device context that owns the library handle
  (Prod/GPU/GPUWrapper.cs:72,99-101,150-160);
* ``GPUTensor``   - shape + raw device pointer, owning or a view
  (Prod/GPU/GpuTensor.cs:13-63); ``Dot`` (:1196-1227) and
  ``BatchMatrixMultiplication`` (:1163-1194) derive M/N/K and leading
  dimensions exactly as the C# does and call the cuBLAS-shaped entry points
  ``snhip_sgemm`` / ``snhip_sgemm_strided_batched`` with the same argument
  order the reference passes to cuBLAS.

All arithmetic happens in libsharpnet_hip.so on the GPU; numpy is used only to
stage host data for the H2D / D2H copies.
"""
import ctypes

import numpy as np

from . import hiplib
from .hiplib import check_status

CUBLAS_OP_N = 0
CUBLAS_OP_T = 1


class GPUWrapper:
    """One per device; owns the library handle, like GPUWrapper owns the cuBLAS handle."""

    _instances = {}

    def __init__(self, device_id=0):
        self.lib = hiplib.load_library()
        self.device_id = device_id
        h = ctypes.c_void_p()
        check_status(self.lib.snhip_create(ctypes.byref(h)), "snhip_create")
        self.handle = h
        self._disposed = False
        self._pool = None   # size in bytes -> released device pointers, when the memory pool is in use

    @classmethod
    def FromDeviceId(cls, device_id=0):
        # GPUWrapper.FromDeviceId caches one wrapper per device (GPUWrapper.cs:150-160)
        w = cls._instances.get(device_id)
        if w is None or w._disposed:
            w = cls(device_id)
            cls._instances[device_id] = w
        return w

    # -- device facts -------------------------------------------------------
    def device_info(self):
        info = (ctypes.c_int * 6)()
        check_status(self.lib.snhip_device_info(self.handle, info), "snhip_device_info")
        return {
            "compute_units": info[0], "clock_khz": info[1], "mem_clock_khz": info[2], "mem_bus_bits": info[3],
            "lds_bytes": info[4], "gfx": info[5],
        }

    def version(self):
        v = ctypes.c_int()
        check_status(self.lib.snhip_get_version(self.handle, ctypes.byref(v)), "snhip_get_version")
        return v.value

    # -- arithmetic ----------------------------------------------------------
    MATH_FP32 = 0
    MATH_BF16_INPUT = 1
    MATH_BF16_STORED = 2

    def set_math_mode(self, mode):
        """fp32 MFMA (default) or bf16-input / fp32-accumulate MFMA for every GEMM of this handle."""
        check_status(self.lib.snhip_set_math_mode(self.handle, mode), "snhip_set_math_mode")

    # -- tuning hooks -------------------------------------------------------
    def set_tuning(self, config=-1, splitk=0):
        check_status(self.lib.snhip_set_tuning(self.handle, config, splitk), "snhip_set_tuning")

    def set_splitk_mode(self, mode):
        """0 automatic, 1 reduce split-K partial sums in a second kernel, 2 in the GEMM kernel."""
        check_status(self.lib.snhip_set_splitk_mode(self.handle, mode), "snhip_set_splitk_mode")

    def last_tuning(self):
        c, s = ctypes.c_int(), ctypes.c_int()
        check_status(self.lib.snhip_get_last_tuning(self.handle, ctypes.byref(c), ctypes.byref(s)))
        return c.value, s.value

    def configs(self):
        out = []
        for i in range(self.lib.snhip_config_count()):
            d = (ctypes.c_int * 6)()
            check_status(self.lib.snhip_config_desc(i, d))
            out.append({"id": i, "BM": d[0], "BN": d[1], "BK": d[2], "threads": d[3], "lds_bytes": d[4],
                        "kind": {0: "fp32", 1: "bf16", 2: "fp32-ksplit", 3: "fp32-stream", 4: "bf16-stored", 5: "bf16-stream",
                                 6: "bf16-stored-stream", 7: "bf16-stored-dtl"}[d[5]]})
        return out

    # -- device memory -------------------------------------------------------
    def use_memory_pool(self, enabled=True):
        """Keep released buffers and hand them out again for requests of the same size, as the reference's
        TensorMemoryPool does for layer buffers (Prod/Data/TensorMemoryPool.cs:59-64: contents are NOT cleared).
        Work on one stream stays ordered, so a reused buffer needs no device synchronisation."""
        if enabled:
            if self._pool is None:
                self._pool = {}
        else:
            self.empty_memory_pool()
            self._pool = None

    def empty_memory_pool(self):
        for ptrs in (self._pool or {}).values():
            while ptrs:
                check_status(self.lib.snhip_free(ptrs.pop()), "snhip_free")

    def allocate(self, nbytes):
        if self._pool is not None and self._pool.get(nbytes):
            return self._pool[nbytes].pop()
        p = ctypes.c_void_p()
        check_status(self.lib.snhip_malloc(ctypes.byref(p), nbytes), "snhip_malloc")
        return p.value

    def release(self, ptr, nbytes):
        if self._pool is not None and not self._disposed:
            self._pool.setdefault(nbytes, []).append(ptr)
        else:
            check_status(self.lib.snhip_free(ptr), "snhip_free")

    # -- stream / timing ----------------------------------------------------
    def synchronize(self):
        check_status(self.lib.snhip_stream_synchronize(self.handle), "snhip_stream_synchronize")

    def new_event(self):
        ev = ctypes.c_void_p()
        check_status(self.lib.snhip_event_create(ctypes.byref(ev)), "snhip_event_create")
        return ev

    def record(self, ev):
        check_status(self.lib.snhip_event_record(self.handle, ev), "snhip_event_record")

    def elapsed_ms(self, start, stop):
        ms = ctypes.c_float()
        check_status(self.lib.snhip_event_elapsed_ms(start, stop, ctypes.byref(ms)), "snhip_event_elapsed_ms")
        return ms.value

    def destroy_event(self, ev):
        check_status(self.lib.snhip_event_destroy(ev), "snhip_event_destroy")

    def Dispose(self):
        if not self._disposed:
            self.empty_memory_pool()
            self._disposed = True
            check_status(self.lib.snhip_destroy(self.handle), "snhip_destroy")
            self.handle = None


def _prod(xs):
    p = 1
    for x in xs:
        p *= int(x)
    return p


class GPUTensor:
    """float32 tensor in device memory (row-major, dense), 1 to 4 dimensions."""

    def __init__(self, shape, data=None, gpu_wrapper=None, _pointer=None, _owner=None):
        shape = [int(s) for s in shape]
        assert 1 <= len(shape) <= 4 and min(shape) >= 0  # Tensor.cs:29-31
        self.Shape = shape
        self.Wrapper = gpu_wrapper or GPUWrapper.FromDeviceId(0)
        self._lib = self.Wrapper.lib
        self._disposed = False
        if _pointer is not None:
            # non-owning view (GpuTensor.cs:52-63)
            self.Pointer = _pointer
            self.IsOwnerOfMemory = False
            self._owner = _owner
        else:
            self.IsOwnerOfMemory = True
            self._owner = None
            self._nbytes = max(self.Count * 4, 8)  # capacity is at least 8 bytes (GpuTensor.cs:38)
            self.Pointer = self.Wrapper.allocate(self._nbytes)
            if data is not None:
                self.InitializeFromHostMemory(data)

    # -- shape helpers (Tensor.cs:18-21,1521-1526) ---------------------------
    @property
    def Count(self):
        return _prod(self.Shape)

    @property
    def Dimension(self):
        return len(self.Shape)

    @property
    def MultDim1(self):
        s = self.Shape
        return s[2] * (s[3] if len(s) >= 4 else 1) if len(s) >= 3 else 1

    @property
    def MultDim0(self):
        s = self.Shape
        return s[1] * self.MultDim1 if len(s) >= 2 else 1

    def AssertIsNotDisposed(self):
        if self._disposed or (self._owner is not None and self._owner._disposed):
            raise RuntimeError("Tensor is disposed")  # GpuTensor.cs:1592-1598

    # -- views ----------------------------------------------------------------
    def Slice(self, startIndex, sliceShape):
        """Non-owning view at element offset startIndex (GpuTensor.cs:616)."""
        self.AssertIsNotDisposed()
        assert startIndex >= 0 and startIndex + _prod(sliceShape) <= self.Count
        return GPUTensor(sliceShape, gpu_wrapper=self.Wrapper, _pointer=self.Pointer + 4 * startIndex,
                         _owner=self._owner or self)

    def RowSlice(self, startRowIndex, nbRows):
        assert len(self.Shape) >= 2 and 0 <= startRowIndex and startRowIndex + nbRows <= self.Shape[0]
        return self.Slice(startRowIndex * self.MultDim0, [nbRows] + self.Shape[1:])

    def GetSubTensor(self, startRowIndex, subTensorShape):
        return self.Slice(startRowIndex * self.MultDim0, subTensorShape)

    def Reshape(self, *newShape):
        newShape = list(newShape)
        if -1 in newShape:
            known = _prod(s for s in newShape if s != -1)
            newShape[newShape.index(-1)] = self.Count // known if known else 0
        assert _prod(newShape) == self.Count
        return GPUTensor(newShape, gpu_wrapper=self.Wrapper, _pointer=self.Pointer, _owner=self._owner or self)

    def As2DTensor(self, flattenInputTensorOnLastDimension):
        # Tensor.cs:1645-1654
        if len(self.Shape) == 2:
            return self
        if flattenInputTensorOnLastDimension:
            return self.Reshape(-1, self.Shape[-1])
        return self.Reshape(self.Shape[0], -1)

    # -- copies ---------------------------------------------------------------
    def InitializeFromHostMemory(self, data):
        self.AssertIsNotDisposed()
        host = np.ascontiguousarray(np.asarray(data, dtype=np.float32).reshape(-1))
        assert host.size == self.Count, "host data has %d elements, tensor has %d" % (host.size, self.Count)
        if host.size:
            check_status(self._lib.snhip_memcpy_htod_async(self.Wrapper.handle, self.Pointer,
                                                           host.ctypes.data, host.nbytes), "snhip_memcpy_htod_async")
            # the staging array must outlive the asynchronous copy
            self.Wrapper.synchronize()

    def ContentAsFloatArray(self):
        """Synchronous D2H copy (GpuTensor.cs:1668)."""
        self.AssertIsNotDisposed()
        host = np.empty(self.Count, dtype=np.float32)
        if host.size:
            check_status(self._lib.snhip_memcpy_dtoh(self.Wrapper.handle, host.ctypes.data, self.Pointer,
                                                     host.nbytes), "snhip_memcpy_dtoh")
        return host

    def ToNumpy(self):
        return self.ContentAsFloatArray().reshape(self.Shape)

    def CopyTo(self, other):
        self.AssertIsNotDisposed()
        other.AssertIsNotDisposed()
        assert other.Count == self.Count
        check_status(self._lib.snhip_memcpy_dtod_async(self.Wrapper.handle, other.Pointer, self.Pointer,
                                                       self.Count * 4), "snhip_memcpy_dtod_async")

    def ZeroMemory(self):
        self.SetValue(0.0)

    def SetValue(self, value):
        self.AssertIsNotDisposed()
        bits = int(np.float32(value).view(np.uint32))
        check_status(self._lib.snhip_memset32(self.Wrapper.handle, self.Pointer, bits, self.Count), "snhip_memset32")

    def Clone(self):
        c = GPUTensor(self.Shape, gpu_wrapper=self.Wrapper)
        self.CopyTo(c)
        return c

    # -- the hot path ----------------------------------------------------------
    def Dot(self, a, transposeA=False, b=None, transposeB=False, alpha=1.0, beta=0.0):
        """this = alpha * op(a) * op(b) + beta * this   (GpuTensor.cs:1196-1227).

        The two-argument form ``c.Dot(a, b)`` is Tensor.cs:60.  Operands with two
        or more dimensions are read as (Shape[0], MultDim0) matrices.
        """
        if b is None or isinstance(transposeA, GPUTensor):
            a, b, transposeA = a, transposeA, False  # c.Dot(a, b)
        self.AssertIsNotDisposed()
        a.AssertIsNotDisposed()
        b.AssertIsNotDisposed()
        assert a.Dimension >= 2 and b.Dimension >= 2 and self.Dimension >= 2
        bH, bW = b.Shape[0], b.MultDim0
        aH, aW = a.Shape[0], a.MultDim0
        transLeft = CUBLAS_OP_T if transposeB else CUBLAS_OP_N
        transRight = CUBLAS_OP_T if transposeA else CUBLAS_OP_N
        N = bH if transposeB else bW
        M = aW if transposeA else aH
        K = bW if transposeB else bH
        ldb, lda, ldc = bW, aW, N
        # column-major library: compute B*A instead of A*B (GpuTensor.cs:1217-1218)
        al, be = ctypes.c_float(alpha), ctypes.c_float(beta)
        res = self._lib.snhip_sgemm(self.Wrapper.handle, transLeft, transRight, N, M, K, ctypes.byref(al),
                                    b.Pointer, ldb, a.Pointer, lda, ctypes.byref(be), self.Pointer, ldc)
        check_status(res, "snhip_sgemm")

    def BatchMatrixMultiplication(self, a_3D, transposeA, b_3D, transposeB, alpha, beta):
        """Strided-batched product of 3-D tensors (GpuTensor.cs:1163-1194)."""
        c_3D = self
        for t in (a_3D, b_3D, c_3D):
            t.AssertIsNotDisposed()
            assert len(t.Shape) == 3
        assert a_3D.Shape[0] == b_3D.Shape[0] == c_3D.Shape[0]
        batchCount = a_3D.Shape[0]
        aH, aW, aStride = a_3D.Shape[1], a_3D.MultDim1, a_3D.MultDim0
        bH, bW, bStride = b_3D.Shape[1], b_3D.MultDim1, b_3D.MultDim0
        cStride = c_3D.MultDim0
        transLeft = CUBLAS_OP_T if transposeB else CUBLAS_OP_N
        transRight = CUBLAS_OP_T if transposeA else CUBLAS_OP_N
        N = bH if transposeB else bW
        M = aW if transposeA else aH
        K = bW if transposeB else bH
        ldb, lda, ldc = bW, aW, N
        al, be = ctypes.c_float(alpha), ctypes.c_float(beta)
        res = self._lib.snhip_sgemm_strided_batched(self.Wrapper.handle, transLeft, transRight, N, M, K,
                                                    ctypes.byref(al), b_3D.Pointer, ldb, bStride, a_3D.Pointer, lda,
                                                    aStride, ctypes.byref(be), self.Pointer, ldc, cStride, batchCount)
        check_status(res, "snhip_sgemm_strided_batched")

    # -- row-major convenience entry points (same numbers, fewer hops) ---------
    def DotRowMajor(self, a, transposeA, b, transposeB, alpha, beta, bias=None):
        """snhip_dot / snhip_dot_bias with BlasServices.DotMkl's parameter list."""
        res = self._lib.snhip_dot_bias(self.Wrapper.handle, a.Pointer, a.Shape[0], a.MultDim0, int(transposeA),
                                       b.Pointer, b.Shape[0], b.MultDim0, int(transposeB), self.Pointer, alpha, beta,
                                       bias.Pointer if bias is not None else None)
        check_status(res, "snhip_dot_bias")

    def GemmEx(self, **fields):
        """snhip_gemm_ex with this tensor as C: keyword arguments are snhip_gemm_desc fields; tensors may be passed
        for A, B, bias, D and colsum (their device pointers are used)."""
        fields = {k: (v.Pointer if isinstance(v, GPUTensor) else v) for k, v in fields.items()}
        desc = hiplib.GemmDesc(C=self.Pointer, **fields)
        check_status(self._lib.snhip_gemm_ex(self.Wrapper.handle, ctypes.byref(desc)), "snhip_gemm_ex")

    # -- lifetime ----------------------------------------------------------------
    def Dispose(self):
        if self._disposed:
            return
        self._disposed = True
        if self.IsOwnerOfMemory and self.Pointer:
            self.Wrapper.release(self.Pointer, self._nbytes)  # GpuTensor.cs:1634 / TensorMemoryPool.FreeFloatTensor
        self.Pointer = None

    def __del__(self):
        try:
            self.Dispose()
        except Exception:
            pass


# -- element-wise / row helpers next to the GEMMs (same names as the reference's Tensor methods) -----------------
def _add_tensor_methods():
    def Compute_BiasGradient_from_dy(self, biasGradient_1D):
        """biasGradient[c] = sum over rows of this[r][c]  (CpuTensor.cs:1736-1740)."""
        assert len(biasGradient_1D.Shape) == 1 and biasGradient_1D.Count == self.MultDim0
        check_status(self._lib.snhip_bias_gradient(self.Wrapper.handle, self.Pointer, self.Shape[0], self.MultDim0,
                                                   biasGradient_1D.Pointer), "snhip_bias_gradient")

    def BroadcastAddVectorToOutput(self, y):
        """y[n, :] += this  (this = 1-D bias; CpuTensor.cs:1468-1487)."""
        assert y.Dimension >= 2 and y.MultDim0 == self.Count
        check_status(self._lib.snhip_broadcast_add_vector(self.Wrapper.handle, self.Pointer, y.Pointer, y.Shape[0],
                                                          y.MultDim0), "snhip_broadcast_add_vector")

    def Update_Adding_Alpha_X(self, alpha, x):
        """this += alpha * x  (Linear.cs:178)."""
        assert x.Count == self.Count
        check_status(self._lib.snhip_axpy(self.Wrapper.handle, self.Count, alpha, x.Pointer, self.Pointer), "snhip_axpy")

    def SoftmaxLastDimension(self, y):
        """y = softmax(this) over the last dimension (ActivationForward(SOFTMAX_LAST_DIMENSION))."""
        cols = self.Shape[-1]
        check_status(self._lib.snhip_softmax_last_dim(self.Wrapper.handle, self.Pointer, y.Pointer,
                                                      self.Count // cols if cols else 0, cols), "snhip_softmax_last_dim")

    def SoftmaxLastDimensionBackward(self, dy, dx):
        """dx = softmax gradient given this = y (ActivationBackward(SOFTMAX_LAST_DIMENSION), cuDNN semantics)."""
        cols = self.Shape[-1]
        check_status(self._lib.snhip_softmax_last_dim_backward(self.Wrapper.handle, self.Pointer, dy.Pointer, dx.Pointer,
                                                               self.Count // cols if cols else 0, cols),
                     "snhip_softmax_last_dim_backward")

    def SetAllElementsAboveMainDiagonal(self, value):
        """CpuTensor.cs:3037-3052; 2-D or 3-D tensors."""
        assert len(self.Shape) in (2, 3)
        m, r, c = (self.Shape if len(self.Shape) == 3 else [1] + self.Shape)
        check_status(self._lib.snhip_set_above_main_diagonal(self.Wrapper.handle, self.Pointer, m, r, c, value),
                     "snhip_set_above_main_diagonal")

    def Transpose(self, transposed):
        """transposed = this^T for a 2-D tensor, through the Sgeam-shaped entry point with the reference's own
        arguments (GpuTensor.cs:1256-1291)."""
        assert self.Dimension == 2 and transposed.Count >= self.Count
        transposed.Shape = [self.Shape[1], self.Shape[0]]
        M, N = self.Shape
        alpha, beta = ctypes.c_float(1.0), ctypes.c_float(0.0)
        check_status(self._lib.snhip_sgeam(self.Wrapper.handle, CUBLAS_OP_T, CUBLAS_OP_N, M, N, ctypes.byref(alpha),
                                           self.Pointer, N, ctypes.byref(beta), None, M, transposed.Pointer, M), "snhip_sgeam")

    def MultiplyTensor(self, a, diagonalMatrix):
        """this = a * diagonalMatrix, element-wise when both have the same size, else every run of
        a.Count / diagonalMatrix.Count consecutive elements scaled by one entry (CpuTensor.cs:1060-1094), through the
        Sdgmm-shaped entry point as the reference calls it (GpuTensor.cs:1380-1395)."""
        assert a.Count == self.Count and self.Count % diagonalMatrix.Count == 0
        n = diagonalMatrix.Count
        m = self.Count // n
        check_status(self._lib.snhip_sdgmm(self.Wrapper.handle, 1, m, n, a.Pointer, m, diagonalMatrix.Pointer, 1,
                                           self.Pointer, m), "snhip_sdgmm")

    def TransposeSecondAndThirdDimension(self, target):
        """target[a][c][b][d] = this[a][b][c][d]; target is reshaped to the swapped shape (CpuTensor.cs:301-322)."""
        assert len(self.Shape) >= 3 and target.Count == self.Count
        A, B, C = self.Shape[:3]
        D = self.Count // max(A * B * C, 1)
        target.Shape = [A, C, B] + list(self.Shape[3:])
        check_status(self._lib.snhip_transpose_second_and_third_dimension(self.Wrapper.handle, self.Pointer, target.Pointer,
                                                                          A, B, C, D),
                     "snhip_transpose_second_and_third_dimension")

    def ActivationForward(self, activationType, activationParameter, y):
        """y = act(this) for the RELU / LEAKY_RELU / SIGMOID / TANH modes (Tensor.ActivationForward);
        activationParameter is the leaky slope."""
        check_status(self._lib.snhip_activation_forward(self.Wrapper.handle, hiplib.activation_code(activationType),
                                                        float(activationParameter or 0.0), self.Pointer, y.Pointer,
                                                        self.Count), "snhip_activation_forward")

    def ActivationBackward(self, activationType, activationParameter, dy, dx):
        """dx = dy * act'(x) with this = y = act(x) (Tensor.ActivationBackward, CPU definitions
        CpuTensorActivationFunctions.cs:190-244)."""
        check_status(self._lib.snhip_activation_backward(self.Wrapper.handle, hiplib.activation_code(activationType),
                                                         float(activationParameter or 0.0), self.Pointer, dy.Pointer,
                                                         dx.Pointer, self.Count), "snhip_activation_backward")

    for f in (Compute_BiasGradient_from_dy, BroadcastAddVectorToOutput, Update_Adding_Alpha_X, SoftmaxLastDimension,
              SoftmaxLastDimensionBackward, SetAllElementsAboveMainDiagonal, Transpose, MultiplyTensor,
              TransposeSecondAndThirdDimension,
              ActivationForward, ActivationBackward):
        setattr(GPUTensor, f.__name__, f)


_add_tensor_methods()
