"""Host-side mirror of TensorSharp.Ops for HipTensor: same op names, argument order and error behaviour as the
reference's static façade (TensorSharp/Ops.cs:15-303) and CPU handlers (TensorSharp/Cpu/CpuBasicOps.cs).

Each function allocates the result when `result` is None (TensorResultBuilder.GetWriteTarget,
TensorSharp/Core/TensorResultBuilder.cs:7-32) and makes exactly one call into libtship.so.
"""
import ctypes as C

import numpy as np

from ._lib import TSHipError, TSHipTensor, check, lib
from .tensor import F16, F32, HipTensor, _protos

ADD, SUB, MUL, DIV = 0, 1, 2, 3
RELU, SILU, LEAKYRELU, EXP, LOG, NEG, SIGMOID, TANH, SQRT, ABS = range(10)

_ok = False


def _p():
    global _ok
    if _ok:
        return lib()
    _protos()
    L = lib()
    T = C.POINTER(TSHipTensor)
    L.TSHip_Copy.argtypes = [T, T]
    L.TSHip_Fill.argtypes = [T, C.c_float]
    L.TSHip_Addmm.argtypes = [T, C.c_float, T, C.c_float, T, T]
    L.TSHip_AddmmBatch.argtypes = [T, C.c_float, T, C.c_float, T, T]
    L.TSHip_IndexSelect.argtypes = [T, T, T, C.c_int]
    L.TSHip_IndexSelectGrad.argtypes = [T, T, T]
    L.TSHip_RoPE.argtypes = [T, T, C.c_int, C.c_int]
    L.TSHip_RoPEEx.argtypes = [T, T, C.c_int, C.c_int, C.c_float]
    L.TSHip_RMSNorm.argtypes = [T, T, T, T, C.c_float]
    L.TSHip_LayerNorm.argtypes = [T, T, T, T, C.c_float]
    L.TSHip_Softmax.argtypes = [T, T]
    L.TSHip_Argmax.argtypes = [T, T, C.c_int]
    L.TSHip_TopK.argtypes = [T, T, T, C.c_int]
    L.TSHip_BinaryTensor.argtypes = [C.c_int, T, T, T]
    L.TSHip_BinaryScalar.argtypes = [C.c_int, T, T, C.c_float]
    L.TSHip_Unary.argtypes = [C.c_int, T, T]
    L.TSHip_BuildTriMask.argtypes = [T, C.c_float, C.c_float]
    L.TSHip_BuildSelfTriMask.argtypes = [T, T, C.c_int, C.c_float, C.c_float]
    L.TSHip_IsCorrupted.argtypes = [T, C.POINTER(C.c_int)]
    L.TSHip_TopPSample.argtypes = [T, T, T, C.c_float]
    L.TSHip_Gather.argtypes = [T, T, C.c_int, T]
    L.TSHip_ScatterFill.argtypes = [T, C.c_float, C.c_int, T]
    L.TSHip_TopPSampleNoAlloc.argtypes = [T, T, T, C.c_float]
    L.TSHip_TopPSampleEx.argtypes = [T, T, T, C.c_float, C.c_float, C.c_void_p, C.c_void_p, C.c_int]
    _ok = True
    return L


def _d(t):
    return None if t is None else C.byref(t.desc())


def _target(result, sizes, dtype, require_contiguous=False):
    """TensorResultBuilder.GetWriteTarget: a supplied result must already have the right size (and layout)."""
    sizes = [int(s) for s in sizes]
    if result is None:
        return HipTensor(sizes, dtype)
    if list(result.sizes) != sizes:
        raise TSHipError("Size mismatch. Received result of size %s, expected %s" % (result.sizes, sizes))
    if require_contiguous and not result.is_contiguous():
        raise TSHipError("Result must be a contiguous tensor")
    return result


def copy(result, src):                                   # "copy"
    check(_p().TSHip_Copy(_d(result), _d(src)))
    return result


def as_contiguous(src):                                  # Ops.AsContiguous, Ops.cs:24-34
    if src.is_contiguous():
        return HipTensor(src.sizes, src.dtype, src.storage, src.strides, src.offset)
    r = HipTensor(src.sizes, src.dtype)
    return copy(r, src)


def fill(result, value):                                 # "fill"
    check(_p().TSHip_Fill(_d(result), float(value)))
    return result


def float2half(result, src):                             # "float2half"
    r = _target(result, src.sizes, F16)
    return copy(r, src)


def half2float(result, src):                             # "half2float"
    r = _target(result, src.sizes, F32)
    return copy(r, src)


def addmm(result, beta, src, alpha, m1, m2):             # "addmm", CpuBasicOps.cs:49-114
    r = _target(result, src.sizes, src.dtype)
    check(_p().TSHip_Addmm(_d(r), float(beta), _d(src), float(alpha), _d(m1), _d(m2)))
    return r


def addmmbatch(result, beta, src, alpha, m1, m2):        # "addmmbatch", CpuBasicOps.cs:116-184
    r = _target(result, src.sizes, src.dtype, True)
    check(_p().TSHip_AddmmBatch(_d(r), float(beta), _d(src), float(alpha), _d(m1), _d(m2)))
    return r


def indexselect(result, src, indice, is_add=False):      # "indexselect", CpuBasicOps.cs:990-1007
    r = _target(result, [indice.sizes[0], src.sizes[1]], src.dtype)
    check(_p().TSHip_IndexSelect(_d(r), _d(src), _d(indice), int(is_add)))
    return r


def indexselectgrad(grad, adj, indice):                  # "indexselectgrad", CpuBasicOps.cs:1010-1030
    if grad is None:
        raise TSHipError("Tensor grad should not be null.")
    check(_p().TSHip_IndexSelectGrad(_d(grad), _d(adj), _d(indice)))
    return grad


def rope(result, src, seq_len, row_offset):              # "rope", CpuBasicOps.cs:1049-1066
    r = _target(result, src.sizes, src.dtype, True)
    check(_p().TSHip_RoPE(_d(r), _d(src), int(seq_len), int(row_offset)))
    return r


def rmsnorm(result, src, alpha, beta, eps):              # "rmsnorm", CpuBasicOps.cs:947-953
    r = _target(result, src.sizes, src.dtype, True)
    check(_p().TSHip_RMSNorm(_d(r), _d(src), _d(alpha), _d(beta), float(eps)))
    return r


def layernorm(result, src, alpha, beta, eps):            # "layernorm"
    r = _target(result, src.sizes, src.dtype, True)
    check(_p().TSHip_LayerNorm(_d(r), _d(src), _d(alpha), _d(beta), float(eps)))
    return r


def softmax(result, src):                                # "softmax", CpuBasicOps.cs:1106-1123
    r = _target(result, src.sizes, src.dtype, True)
    check(_p().TSHip_Softmax(_d(r), _d(src)))
    return r


def argmax(result, src, dim):                            # "argmax", CpuBasicOps.cs:832-840
    sizes = list(src.sizes)
    sizes[dim] = 1
    r = _target(result, sizes, F32)
    check(_p().TSHip_Argmax(_d(r), _d(src), int(dim)))
    return r


def topk(out_val, out_idx, src, k):                      # "topK", CpuBasicOps.cs:1032-1047
    sizes = list(src.sizes)
    sizes[-1] = k
    ov = _target(out_val, sizes, src.dtype)
    oi = _target(out_idx, sizes, F32)
    check(_p().TSHip_TopK(_d(ov), _d(oi), _d(src), int(k)))
    return ov, oi


def _binary(op, result, lhs, rhs):
    r = _target(result, lhs.sizes, lhs.dtype)
    check(_p().TSHip_BinaryTensor(op, _d(r), _d(lhs), _d(rhs)))
    return r


def add(result, lhs, rhs):                               # "addt" / "addv"
    if isinstance(rhs, HipTensor):
        return _binary(ADD, result, lhs, rhs)
    return _scalar(ADD, result, lhs, rhs)


def sub(result, lhs, rhs):
    if isinstance(rhs, HipTensor):
        return _binary(SUB, result, lhs, rhs)
    return _scalar(SUB, result, lhs, rhs)


def mul(result, lhs, rhs):                               # "mult" / "mulv"
    if isinstance(rhs, HipTensor):
        return _binary(MUL, result, lhs, rhs)
    return _scalar(MUL, result, lhs, rhs)


def div(result, lhs, rhs):                               # "divt" / "divv"
    if isinstance(rhs, HipTensor):
        return _binary(DIV, result, lhs, rhs)
    return _scalar(DIV, result, lhs, rhs)


def _scalar(op, result, src, value):
    r = _target(result, src.sizes, src.dtype)
    check(_p().TSHip_BinaryScalar(op, _d(r), _d(src), float(value)))
    return r


def _unary(op, result, src):
    r = _target(result, src.sizes, src.dtype)
    check(_p().TSHip_Unary(op, _d(r), _d(src)))
    return r


def relu(result, src):
    return _unary(RELU, result, src)


def silu(result, src):                                   # "SiLU"
    return _unary(SILU, result, src)


def leakyrelu(result, src):                              # "LeakyReLU"
    return _unary(LEAKYRELU, result, src)


def exp(result, src):
    return _unary(EXP, result, src)


def log(result, src):
    return _unary(LOG, result, src)


def sigmoid(result, src):
    return _unary(SIGMOID, result, src)


def neg(result, src):
    return _unary(NEG, result, src)


def tanh(result, src):
    return _unary(TANH, result, src)


def sqrt(result, src):
    return _unary(SQRT, result, src)


def abs(result, src):                                    # "abs" (the op registry's name)
    return _unary(ABS, result, src)


def buildtrimask(result, value, masked_value):           # "buildtrimask"
    check(_p().TSHip_BuildTriMask(_d(result), float(value), float(masked_value)))
    return result


def buildselftrimask(result, original_lengths, padded_seq_len, value, masked_value):
    check(_p().TSHip_BuildSelfTriMask(_d(result), _d(original_lengths), int(padded_seq_len), float(value), float(masked_value)))
    return result


def iscorrupted(src):                                    # "iscorrupted"
    flag = C.c_int(0)
    check(_p().TSHip_IsCorrupted(_d(src), C.byref(flag)))
    return bool(flag.value)


def gather(result, src, dim, indices):                   # "gather", CpuIndexingOps.cs:23-56
    r = _target(result, indices.sizes, src.dtype)
    check(_p().TSHip_Gather(_d(r), _d(src), int(dim), _d(indices)))
    return r


def scatter_fill(result, value, dim, indices):           # "scatter_fill", CpuIndexingOps.cs:141-167
    check(_p().TSHip_ScatterFill(_d(result), float(value), int(dim), _d(indices)))
    return result


def toppsample(result, probs, uniforms, top_p, repeat_penalty=0.0, seqs=None, seq_lens=None):
    """ComputeGraphTensor.TopPSample (Seq2SeqSharp/Tools/ComputeGraphTensor.cs:2305-2403); `seqs` = decodedSequences as an
    int32 array [rows, max_len] (with `seq_lens` [rows] when the rows differ in length), None = no decay."""
    r = _target(result, [probs.sizes[0], 1], F32)
    if seqs is None:
        check(_p().TSHip_TopPSample(_d(r), _d(probs), _d(uniforms), float(top_p)))
        return r
    seqs = np.ascontiguousarray(seqs, dtype=np.int32)
    lens = np.full((seqs.shape[0],), seqs.shape[1], np.int32) if seq_lens is None else np.ascontiguousarray(seq_lens, dtype=np.int32)
    check(_p().TSHip_TopPSampleEx(_d(r), _d(probs), _d(uniforms), float(top_p), float(repeat_penalty),
                                  seqs.ctypes.data_as(C.c_void_p), lens.ctypes.data_as(C.c_void_p), int(seqs.shape[1])))
    return r


def toppsample_noalloc(result, probs, uniforms, top_p):
    """TSHip_TopPSample on the library's fixed scratch array: nothing is allocated, so `result` must be supplied.  Not
    synchronised: read the result after a synchronising call (HipTensor.numpy does)."""
    check(_p().TSHip_TopPSampleNoAlloc(_d(result), _d(probs), _d(uniforms), float(top_p)))
    return result


def concat(dim, tensors):
    """TensorConcatenation.Concat (TensorSharp/Core/TensorConcatenation.cs:9-45): a new tensor, inputs copied in order."""
    sizes = list(tensors[0].sizes)
    sizes[dim] = sum(t.sizes[dim] for t in tensors)
    r = HipTensor(sizes, tensors[0].dtype)
    at = 0
    for t in tensors:
        v = r.narrow(dim, at, t.sizes[dim])
        copy(v, t)
        v.dispose()
        at += t.sizes[dim]
    return r
