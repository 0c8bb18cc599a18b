"""Host-side mirror of TensorSharp's data model for the HIP backend: storage, allocator, strided tensor views.

Mirrors TensorSharp/Tensor.cs:12-440 (sizes and strides in elements, zero-copy View / Narrow / Select /
Transpose / Expand), TensorSharp/Storage.cs:7-48 and TensorSharp/IAllocator.cs:13-20.  Device memory comes
from the C ABI (TSHip_Malloc / TSHip_Free); host<->device copies are synchronous like CudaStorage's
(TensorSharp.CUDA/CudaStorage.cs:35-173).
"""
import ctypes as C

import numpy as np

from ._lib import MAX_DIMS, TSHipError, TSHipTensor, check, lib

F32, F16 = 0, 1            # TensorSharp/DType.cs:6-13
_NP = {F32: np.float32, F16: np.float16}
_SZ = {F32: 4, F16: 2}

_ready = False


def _protos():
    global _ready
    if _ready:
        return
    L = lib()
    L.TSHip_Init.argtypes = [C.c_int]
    L.TSHip_Malloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
    L.TSHip_Free.argtypes = [C.c_void_p]
    L.TSHip_MemcpyH2D.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
    L.TSHip_MemcpyD2H.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
    L.TSHip_MemcpyD2D.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
    L.TSHip_Memset.argtypes = [C.c_void_p, C.c_int, C.c_size_t]
    L.TSHip_GetMemInfo.argtypes = [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]
    check(L.TSHip_Init(0))
    _ready = True


class HipStorage:
    """Storage (TensorSharp/Storage.cs): a refcounted device buffer of `element_count` elements."""

    def __init__(self, dtype, element_count):
        _protos()
        self.dtype = dtype
        self.element_count = int(element_count)
        p = C.c_void_p()
        check(lib().TSHip_Malloc(C.byref(p), max(1, self.element_count) * _SZ[dtype]))
        self.ptr = p.value
        self.refs = 1

    def add_ref(self):
        self.refs += 1

    def release(self):
        self.refs -= 1
        if self.refs == 0 and self.ptr:
            lib().TSHip_Free(C.c_void_p(self.ptr))     # Storage.Destroy at refcount zero
            self.ptr = None

    def __del__(self):
        try:
            if self.ptr:
                lib().TSHip_Free(C.c_void_p(self.ptr))
                self.ptr = None
        except Exception:
            pass

    # Storage.CopyToStorage / CopyFromStorage / Get|SetElementsAsFloat (linear, strides ignored)
    def copy_to_storage(self, index, host_array):
        a = np.ascontiguousarray(host_array, dtype=_NP[self.dtype])
        if index < 0 or index + a.size > self.element_count:
            raise TSHipError("CopyToStorage: range outside the storage")
        check(lib().TSHip_MemcpyH2D(C.c_void_p(self.ptr + index * _SZ[self.dtype]), a.ctypes.data_as(C.c_void_p), a.nbytes))

    def copy_from_storage(self, index, count):
        if index < 0 or index + count > self.element_count:
            raise TSHipError("CopyFromStorage: range outside the storage")
        out = np.empty((count,), _NP[self.dtype])
        if count:
            check(lib().TSHip_MemcpyD2H(out.ctypes.data_as(C.c_void_p), C.c_void_p(self.ptr + index * _SZ[self.dtype]), out.nbytes))
        return out

    def location_description(self):
        return "HIP:0"


class HipAllocator:
    """IAllocator (TensorSharp/IAllocator.cs:13-20)."""
    device_id = 0

    def allocate(self, dtype, element_count):
        return HipStorage(dtype, element_count)

    def get_allocated_memory_ratio(self):
        _protos()
        f, t = C.c_size_t(0), C.c_size_t(0)
        check(lib().TSHip_GetMemInfo(C.byref(f), C.byref(t)))
        return 1.0 - f.value / float(t.value)


def _contig_strides(sizes):
    st, s = [], 1
    for n in reversed(sizes):
        st.append(s)
        s *= n
    return list(reversed(st))


class HipTensor:
    """Tensor (TensorSharp/Tensor.cs): sizes, strides (elements), storage, storage offset."""

    def __init__(self, sizes, dtype=F32, storage=None, strides=None, offset=0):
        self.sizes = [int(s) for s in sizes]
        self.dtype = dtype
        self.strides = [int(s) for s in (strides if strides is not None else _contig_strides(self.sizes))]
        self.offset = int(offset)
        if storage is None:
            n = 1
            for s in self.sizes:
                n *= s
            storage = HipStorage(dtype, n)
        else:
            storage.add_ref()
        self.storage = storage
        if len(self.sizes) > MAX_DIMS:
            raise TSHipError("tensors of more than %d dimensions are not supported" % MAX_DIMS)

    # ---- construction from / to host -----------------------------------------------------------------
    @staticmethod
    def from_numpy(a, dtype=None):
        a = np.asarray(a)
        if dtype is None:
            dtype = F16 if a.dtype == np.float16 else F32
        t = HipTensor(a.shape if a.ndim else (1,), dtype)
        t.storage.copy_to_storage(0, a.reshape(-1))
        return t

    def numpy(self):
        """The logical contents as a float32 array (a contiguous device copy is made for strided views)."""
        src = self
        if not self.is_contiguous():
            from . import ops
            src = ops.as_contiguous(self)
        n = src.element_count()
        out = src.storage.copy_from_storage(src.offset, n).astype(np.float32).reshape(self.sizes)
        return out

    def dispose(self):
        if self.storage is not None:
            self.storage.release()
            self.storage = None

    # ---- shape algebra (zero-copy) ---------------------------------------------------------------------
    def element_count(self):
        n = 1
        for s in self.sizes:
            n *= s
        return n

    def is_contiguous(self):                      # Tensor.IsContiguous, Tensor.cs:254-268
        s = 1
        for n, st in zip(reversed(self.sizes), reversed(self.strides)):
            if st != s:
                return False
            s *= n
        return True

    def _like(self, sizes, strides, offset=None):
        return HipTensor(sizes, self.dtype, self.storage, strides, self.offset if offset is None else offset)

    def view(self, *sizes):                       # Tensor.View, Tensor.cs:295-312
        if not self.is_contiguous():
            raise TSHipError("Cannot use View on a non-contiguous tensor")
        sizes = list(sizes[0]) if len(sizes) == 1 and isinstance(sizes[0], (list, tuple)) else list(sizes)
        n = self.element_count()
        if -1 in sizes:
            known = 1
            for s in sizes:
                if s != -1:
                    known *= s
            sizes[sizes.index(-1)] = n // known
        m = 1
        for s in sizes:
            m *= s
        if m != n:
            raise TSHipError("Output tensor must have the same number of elements as the input")
        return self._like(sizes, _contig_strides(sizes))

    def transpose(self, d1=0, d2=1):              # Tensor.Transpose, Tensor.cs:380-400
        sz, st = list(self.sizes), list(self.strides)
        sz[d1], sz[d2] = sz[d2], sz[d1]
        st[d1], st[d2] = st[d2], st[d1]
        return self._like(sz, st)

    def expand(self, *sizes):                     # Tensor.Expand, Tensor.cs:415-440
        sizes = list(sizes[0]) if len(sizes) == 1 and isinstance(sizes[0], (list, tuple)) else list(sizes)
        if len(sizes) != len(self.sizes):
            raise TSHipError("number of dimensions of newSizes must equal the tensor's")
        st = list(self.strides)
        for i, (o, n) in enumerate(zip(self.sizes, sizes)):
            if o != n:
                if o != 1:
                    raise TSHipError("Can only expand singleton dimensions")
                st[i] = 0
        return self._like(sizes, st)

    def narrow(self, dim, start, size):           # Tensor.Narrow, Tensor.cs:330-352
        if start < 0 or start + size > self.sizes[dim]:
            raise TSHipError("narrow: range out of bounds")
        sz = list(self.sizes)
        sz[dim] = size
        return self._like(sz, self.strides, self.offset + start * self.strides[dim])

    def select(self, dim, index):                 # Tensor.Select, Tensor.cs:354-372
        t = self.narrow(dim, index, 1)
        sz, st = list(t.sizes), list(t.strides)
        del sz[dim], st[dim]
        r = self._like(sz, st, t.offset)
        t.dispose()
        return r

    # ---- C ABI descriptor ---------------------------------------------------------------------------------
    def desc(self):
        d = TSHipTensor()
        d.data = self.storage.ptr + self.offset * _SZ[self.dtype]
        d.dtype = self.dtype
        d.ndim = len(self.sizes)
        for i in range(MAX_DIMS):
            d.sizes[i] = self.sizes[i] if i < d.ndim else 1
            d.strides[i] = self.strides[i] if i < d.ndim else 0
        return d
