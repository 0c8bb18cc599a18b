// Per-op surface of the C ABI: one entry point per OpRegistry name that the GPTDecoder layers issue
// (TensorSharp/Ops.cs:15-303; CPU handlers in TensorSharp/Cpu/CpuBasicOps.cs, arithmetic in
// TensorSharp/TensorApplyCPU.cs).  These make Seq2SeqSharp's unmodified layer code runnable on the device;
// they accept arbitrary strided views (Expand = stride 0, Transpose, Narrow) in fp32 or fp16.  The fused path in
// tship_gpt.hip is what the benchmark measures; this surface is about same names, same signatures, same results.
#include "tship_internal.h"
#include "tship_sample_kernels.h"

#include <cstring>
#include <functional>
#include <vector>

namespace tship {

// Scratch of TSHip_TopPSampleNoAlloc, the entry point that allocates nothing: sort keys, indices, running sums and digit
// counts of the top-p pipeline.  Every GPU the library runs on holds its own copy of this array, at its own address, until
// the process ends.  In host code the array's name is only a stand-in for that address: the address is asked for once per
// device at initialisation (noalloc_device_setup) and only that pointer is ever handed to kernels.
constexpr size_t NOALLOC_SCRATCH_BYTES = 6u << 20;
static __device__ __align__(256) unsigned char scratch[NOALLOC_SCRATCH_BYTES];
constexpr int NOALLOC_MAX_DEVICES = 64;
static unsigned char* g_scratch_ptr[NOALLOC_MAX_DEVICES] = {};

// called by TSHip_Init with `device` current
void noalloc_device_setup(int device) {
    TSHIP_REQUIRE(device >= 0 && device < NOALLOC_MAX_DEVICES, "TSHip_Init: device id beyond the per-device scratch table");
    if (g_scratch_ptr[device]) return;
    unsigned char* ptr = nullptr;
    TSHIP_CHECK_HIP(hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)));
    TSHIP_REQUIRE(ptr != nullptr, "TSHip_Init: the device scratch array has no address");
    g_scratch_ptr[device] = ptr;
}

struct View {
    void* p; int dtype; int nd;
    long sz[TSHIP_MAX_DIMS]; long st[TSHIP_MAX_DIMS];
};

static View make_view(const TSHipTensor* t, const char* what) {
    if (!t) throw Error(std::string(what) + ": tensor argument is null");
    if (!t->data) throw Error(std::string(what) + ": tensor data pointer is null");
    if (t->ndim < 1 || t->ndim > TSHIP_MAX_DIMS) throw Error(std::string(what) + ": ndim out of range");
    if (t->dtype != TSHIP_F32 && t->dtype != TSHIP_F16) throw Error(std::string(what) + ": only Float32 and Float16 tensors are supported");
    View v; v.p = t->data; v.dtype = t->dtype; v.nd = t->ndim;
    for (int i = 0; i < TSHIP_MAX_DIMS; ++i) { v.sz[i] = 1; v.st[i] = 0; }
    for (int i = 0; i < t->ndim; ++i) {
        if (t->sizes[i] < 0) throw Error(std::string(what) + ": negative size");
        if (t->strides[i] < 0) throw Error(std::string(what) + ": negative strides are not supported");
        v.sz[i] = t->sizes[i]; v.st[i] = t->strides[i];
    }
    return v;
}
static long count(const View& v) { long c = 1; for (int i = 0; i < v.nd; ++i) c *= v.sz[i]; return c; }
static bool same_shape(const View& a, const View& b) {
    if (a.nd != b.nd) return false;
    for (int i = 0; i < a.nd; ++i) if (a.sz[i] != b.sz[i]) return false;
    return true;
}
static bool is_contiguous(const View& v) {
    long s = 1;
    for (int i = v.nd - 1; i >= 0; --i) { if (v.sz[i] != 1 && v.st[i] != s) return false; s *= v.sz[i]; }
    return true;
}
// collapse all dims but the last into "rows": a view usable by the row kernels
struct RowView { void* p; int dtype; int nd; long sz[TSHIP_MAX_DIMS]; long st[TSHIP_MAX_DIMS]; long rows, cols, cstride; };
static RowView row_view(const View& v) {
    RowView r; r.p = v.p; r.dtype = v.dtype; r.nd = v.nd - 1;
    r.cols = v.sz[v.nd - 1]; r.cstride = v.st[v.nd - 1]; r.rows = 1;
    for (int i = 0; i < TSHIP_MAX_DIMS; ++i) { r.sz[i] = 1; r.st[i] = 0; }
    for (int i = 0; i < v.nd - 1; ++i) { r.sz[i] = v.sz[i]; r.st[i] = v.st[i]; r.rows *= v.sz[i]; }
    return r;
}

__device__ __forceinline__ long view_offset(const View& v, long lin) {
    long off = 0;
#pragma unroll
    for (int i = TSHIP_MAX_DIMS - 1; i >= 0; --i) {
        if (i < v.nd) { long q = lin / v.sz[i]; off += (lin - q * v.sz[i]) * v.st[i]; lin = q; }
    }
    return off;
}
__device__ __forceinline__ long row_offset(const RowView& v, long row) {
    long off = 0;
#pragma unroll
    for (int i = TSHIP_MAX_DIMS - 1; i >= 0; --i) {
        if (i < v.nd) { long q = row / v.sz[i]; off += (row - q * v.sz[i]) * v.st[i]; row = q; }
    }
    return off;
}
__device__ __forceinline__ float ld(const void* p, int dtype, long off) {
    return dtype == TSHIP_F16 ? (float)((const half_t*)p)[off] : ((const float*)p)[off];
}
__device__ __forceinline__ void st(void* p, int dtype, long off, float v) {
    if (dtype == TSHIP_F16) ((half_t*)p)[off] = (half_t)v; else ((float*)p)[off] = v;
}

// ---- element-wise ------------------------------------------------------------------------------
enum { EW_COPY = 100, EW_FILL = 101 };

__device__ __forceinline__ float unary_apply(int op, float w) {
    // TensorSharp/TensorApplyCPU.cs:1747-1801 for the activations
    switch (op) {
        case TSHIP_RELU: return w < 0.0f ? 0.0f : w;
        case TSHIP_SILU: return w / (1.0f + expf(-w));
        case TSHIP_LEAKYRELU: return w < 0.0f ? 0.01f * w : w;
        case TSHIP_EXP: return expf(w);
        case TSHIP_LOG: return logf(w);
        case TSHIP_NEG: return -w;
        case TSHIP_SIGMOID: return 1.0f / (1.0f + expf(-w));
        case TSHIP_TANH: return tanhf(w);
        case TSHIP_SQRT: return sqrtf(w);
        case TSHIP_ABS: return fabsf(w);
        default: return w;
    }
}
__device__ __forceinline__ float binary_apply(int op, float a, float b) {
    switch (op) {
        case TSHIP_ADD: return a + b;
        case TSHIP_SUB: return a - b;
        case TSHIP_MUL: return a * b;
        default: return a / b;
    }
}

__global__ void ew_unary_kernel(View r, View s, int op, long n) {
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float v = ld(s.p, s.dtype, view_offset(s, i));
    st(r.p, r.dtype, view_offset(r, i), op == EW_COPY ? v : unary_apply(op, v));
}
__global__ void ew_fill_kernel(View r, float value, long n) {
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    st(r.p, r.dtype, view_offset(r, i), value);
}
__global__ void ew_binary_kernel(View r, View a, View b, int op, long n) {
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    st(r.p, r.dtype, view_offset(r, i), binary_apply(op, ld(a.p, a.dtype, view_offset(a, i)), ld(b.p, b.dtype, view_offset(b, i))));
}
__global__ void ew_scalar_kernel(View r, View a, float s, int op, long n) {
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    st(r.p, r.dtype, view_offset(r, i), binary_apply(op, ld(a.p, a.dtype, view_offset(a, i)), s));
}

// ---- gather / scatter_fill along one dimension (TensorApplyCPU.cs:200-257 through ApplyDim2 / ApplyDim3) -------------
// One thread per element of `indices`.  gather: result[.., j, ..] = src[.., (long)indices[.., j, ..], ..];
// scatter_fill: result[.., (long)indices[.., j, ..], ..] = value.  An index outside the dimension (the reference throws
// IndexOutOfRangeException) sets *bad and is skipped.
__global__ void gather_kernel(View r, View s, View ix, int dim, long n, int* bad) {
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const long idx = (long)ld(ix.p, ix.dtype, view_offset(ix, i));
    if (idx < 0 || idx >= s.sz[dim]) { *bad = 1; return; }
    long lin = i, so = 0;
#pragma unroll
    for (int d = TSHIP_MAX_DIMS - 1; d >= 0; --d) {
        if (d < ix.nd) { const long q = lin / ix.sz[d]; const long c = lin - q * ix.sz[d]; so += (d == dim ? idx : c) * s.st[d]; lin = q; }
    }
    st(r.p, r.dtype, view_offset(r, i), ld(s.p, s.dtype, so));
}
__global__ void scatter_fill_kernel(View r, View ix, int dim, float value, long n, int* bad) {
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const long idx = (long)ld(ix.p, ix.dtype, view_offset(ix, i));
    if (idx < 0 || idx >= r.sz[dim]) { *bad = 1; return; }
    long lin = i, ro = 0;
#pragma unroll
    for (int d = TSHIP_MAX_DIMS - 1; d >= 0; --d) {
        if (d < ix.nd) { const long q = lin / ix.sz[d]; const long c = lin - q * ix.sz[d]; ro += (d == dim ? idx : c) * r.st[d]; lin = q; }
    }
    st(r.p, r.dtype, ro, value);
}

// ---- GEMM over strided 2-D views, optional batch (blockIdx.z) ---------------------------------------
struct MatView { void* p; int dtype; long s0, s1, sb; };
__global__ __launch_bounds__(256) void gemm_strided_kernel(MatView C, MatView S, MatView A, MatView B, int M, int N, int K, float alpha, float beta) {
    __shared__ float As[16][64 + 4];
    __shared__ float Bs[16][64 + 4];
    const int t = threadIdx.x, tx = t & 15, ty = t >> 4;
    const int col0 = blockIdx.x * 64, row0 = blockIdx.y * 64; const long bz = blockIdx.z;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.0f;
    const int am = t >> 2, ak = (t & 3) * 4, bk = t >> 4, bn = (t & 15) * 4;
    for (int k0 = 0; k0 < K; k0 += 16) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            int r = row0 + am, k = k0 + ak + j;
            As[ak + j][am] = (r < M && k < K) ? ld(A.p, A.dtype, bz * A.sb + (long)r * A.s0 + (long)k * A.s1) : 0.0f;
            int kk = k0 + bk, c = col0 + bn + j;
            Bs[bk][bn + j] = (kk < K && c < N) ? ld(B.p, B.dtype, bz * B.sb + (long)kk * B.s0 + (long)c * B.s1) : 0.0f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < 16; ++k) {
            float av[4], bv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) { av[i] = As[k][ty * 4 + i]; bv[i] = Bs[k][tx * 4 + i]; }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], bv[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        int r = row0 + ty * 4 + i;
        if (r >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            int c = col0 + tx * 4 + j;
            if (c >= N) continue;
            float v = alpha * acc[i][j];
            if (beta != 0.0f) v += beta * ld(S.p, S.dtype, bz * S.sb + (long)r * S.s0 + (long)c * S.s1);
            st(C.p, C.dtype, bz * C.sb + (long)r * C.s0 + (long)c * C.s1, v);
        }
    }
}

// ---- GEMM on the matrix cores for fp16 operands with contiguous rows (what Affine and Mul issue on fp16 models) -------
// C[M,N] = beta * S + alpha * A[M,K] B[K,N], fp32 accumulation.  Block tile 128 x 64, four wavefronts, each a 32-row
// strip of the tile and both of its 32-column halves; k advances 16 per step with v_mfma_f32_32x32x16_f16:
//   A operand (32 rows x 16 k): lane l holds row l % 32, k = 8 (l / 32) .. + 7: 16 contiguous bytes of a row of A, read
//     straight from global memory;
//   B operand (16 k x 32 columns): lane l holds column l % 32, k = 8 (l / 32) .. + 7, a column walk in row-major B: the
//     block stages the 16 x 64 tile of B in LDS transposed ([column][k], two stages), so that a lane reads its 8 values
//     as one 16-byte LDS load;
//   D: lane l, register v holds row 8 (v / 4) + 4 (l / 32) + v % 4, column l % 32: a register is a run of 32 columns.
// The host takes this path when K % 8 == 0, N % 4 == 0, the leading dimensions keep 16-byte (A) and 8-byte (B) alignment
// and inner strides are 1; everything else goes to the generic kernel above.
__global__ __launch_bounds__(256) void gemm_f16_mfma_kernel(MatView C, MatView S, MatView A, MatView B, int M, int N, int K, float alpha, float beta) {
    __shared__ __attribute__((aligned(16))) half_t Bs[2][64][24];        // [stage][column][k (16, padded to 24: conflict-free 16-byte reads)]
    const int t = threadIdx.x, lane = t & 63, w = t >> 6;
    const int col0 = blockIdx.x * 64, row0 = blockIdx.y * 128 + w * 32; const long bz = blockIdx.z;
    const half_t* Ab = (const half_t*)A.p + bz * A.sb;
    const half_t* Bb = (const half_t*)B.p + bz * B.sb;
    floatx16 acc[2];
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[j][v] = 0.0f;
    const int am = row0 + (lane & 31), ak = 8 * (lane >> 5);
    const bool a_ok = am < M;
    // staging of B: thread t brings 4 columns of one k row
    const int bk = t >> 4, bn = (t & 15) * 4;
    const bool b_ok = col0 + bn < N;            // (N is a multiple of 4: a group of 4 columns is inside or outside)
    const int nk = (K + 15) / 16;
    auto stage_b = [&](int kt, int st) {
        half4 v = half4{0, 0, 0, 0};
        const int k = kt * 16 + bk;
        if (b_ok && k < K) v = *(const half4*)(Bb + (long)k * B.s0 + col0 + bn);
#pragma unroll
        for (int i = 0; i < 4; ++i) Bs[st][bn + i][bk] = v[i];
    };
    stage_b(0, 0);
    for (int kt = 0; kt < nk; ++kt) {
        half8 af = half8{0, 0, 0, 0, 0, 0, 0, 0};
        if (a_ok && kt * 16 + ak < K) af = *(const half8*)(Ab + (long)am * A.s0 + kt * 16 + ak);      // (K is a multiple of 8)
        __syncthreads();                        // stage kt & 1 is complete; the other one has been consumed
        if (kt + 1 < nk) stage_b(kt + 1, (kt + 1) & 1);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const half8 bf = *(const half8*)(&Bs[kt & 1][j * 32 + (lane & 31)][ak]);
            acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af, bf, acc[j], 0, 0, 0);
        }
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int c = col0 + j * 32 + (lane & 31);
        if (c >= N) continue;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int r = row0 + 8 * (v / 4) + 4 * (lane >> 5) + (v % 4);
            if (r >= M) continue;
            float o = alpha * acc[j][v];
            if (beta != 0.0f) o += beta * ld(S.p, S.dtype, bz * S.sb + (long)r * S.s0 + (long)c * S.s1);
            ((half_t*)C.p)[bz * C.sb + (long)r * C.s0 + c] = (half_t)o;
        }
    }
}

// ---- row kernels: one 256-thread block per row ----------------------------------------------------
__global__ __launch_bounds__(256) void softmax_rows_kernel(RowView r, RowView s) {
    __shared__ float sred[4];
    const long row = blockIdx.x; const int t = threadIdx.x;
    const long so = row_offset(s, row), ro = row_offset(r, row);
    float mx = -INFINITY;
    for (long c = t; c < s.cols; c += 256) mx = fmaxf(mx, ld(s.p, s.dtype, so + c * s.cstride));
    mx = block_max_256(mx, sred);
    float sum = 0.0f;
    for (long c = t; c < s.cols; c += 256) sum += expf(ld(s.p, s.dtype, so + c * s.cstride) - mx);
    sum = block_sum_256(sum, sred);
    for (long c = t; c < s.cols; c += 256) st(r.p, r.dtype, ro + c * r.cstride, expf(ld(s.p, s.dtype, so + c * s.cstride) - mx) / sum);
}

__global__ __launch_bounds__(256) void norm_rows_kernel(RowView r, RowView s, const void* gamma, int gdt, long gs, const void* beta, int bdt, long bs,
                                                        float eps, int layer) {
    __shared__ float sred[4];
    const long row = blockIdx.x; const int t = threadIdx.x;
    const long so = row_offset(s, row), ro = row_offset(r, row);
    const float n = (float)s.cols;
    float sum = 0.0f, sq = 0.0f;
    for (long c = t; c < s.cols; c += 256) { float v = ld(s.p, s.dtype, so + c * s.cstride); sum += v; sq += v * v; }
    if (!layer) {
        // TensorApplyCPU.RMSNorm, TensorApplyCPU.cs:1451-1496
        float rms = sqrtf(block_sum_256(sq, sred) / n + eps);
        for (long c = t; c < s.cols; c += 256) {
            float y = ld(gamma, gdt, c * gs) * (ld(s.p, s.dtype, so + c * s.cstride) / rms);
            if (beta) y += ld(beta, bdt, c * bs);
            st(r.p, r.dtype, ro + c * r.cstride, y);
        }
    } else {
        // TensorApplyCPU.LayerNorm, TensorApplyCPU.cs:1360-1447
        float mean = block_sum_256(sum, sred) / n;
        float d2 = 0.0f;
        for (long c = t; c < s.cols; c += 256) { float d = ld(s.p, s.dtype, so + c * s.cstride) - mean; d2 += d * d; }
        float sigma = sqrtf(eps + block_sum_256(d2, sred) / n);
        for (long c = t; c < s.cols; c += 256) {
            float y = ld(gamma, gdt, c * gs) * ((ld(s.p, s.dtype, so + c * s.cstride) - mean) / sigma);
            if (beta) y += ld(beta, bdt, c * bs);
            st(r.p, r.dtype, ro + c * r.cstride, y);
        }
    }
}

// first maximum wins (TensorApplyCPU.cs:345-355)
__global__ __launch_bounds__(256) void argmax_rows_kernel(RowView r, RowView s) {
    __shared__ float sv[4]; __shared__ long si[4];
    const long row = blockIdx.x; const int t = threadIdx.x;
    const long so = row_offset(s, row);
    // NaN never wins a comparison in the reference's scan; equal values keep the lowest index
    const long NONE = 0x7fffffffffffffffL;
    float best = -INFINITY; long bi = NONE;
    for (long c = t; c < s.cols; c += 256) {
        float v = ld(s.p, s.dtype, so + c * s.cstride);
        if (v > best || (v == best && c < bi)) { best = v; bi = c; }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        float ov = __shfl_xor(best, o, 64); long oi = __shfl_xor(bi, o, 64);
        if (ov > best || (ov == best && oi < bi)) { best = ov; bi = oi; }
    }
    if ((t & 63) == 0) { sv[t >> 6] = best; si[t >> 6] = bi; }
    __syncthreads();
    if (t == 0) {
        for (int w = 1; w < 4; ++w)
            if (sv[w] > best || (sv[w] == best && si[w] < bi)) { best = sv[w]; bi = si[w]; }
        // the reference starts from element 0 and only moves on a strict '>': a NaN there, or a row of NaNs, stays at 0
        float first = ld(s.p, s.dtype, so);
        if (!(first == first) || bi == NONE) bi = 0;
        st(r.p, r.dtype, row_offset(r, row), (float)bi);
    }
}

// one thread per row: the reference's insertion rule, TensorApplyCPU.cs:1099-1146
__global__ void topk_rows_kernel(RowView ov, RowView oi, RowView s, int k) {
    long row = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (row >= s.rows) return;
    const long so = row_offset(s, row), vo = row_offset(ov, row), io = row_offset(oi, row);
    for (int i = 0; i < k; ++i) { st(ov.p, ov.dtype, vo + i * ov.cstride, -1.70141e+38f); st(oi.p, oi.dtype, io + i * oi.cstride, -1.70141e+38f); }
    for (long c = 0; c < s.cols; ++c) {
        float data = ld(s.p, s.dtype, so + c * s.cstride);
        if (data < ld(ov.p, ov.dtype, vo + (k - 1) * ov.cstride)) continue;
        int j = k - 2;
        for (; j >= 0; --j) {
            float aj = ld(ov.p, ov.dtype, vo + j * ov.cstride);
            if (data > aj) {
                st(ov.p, ov.dtype, vo + (j + 1) * ov.cstride, aj);
                st(oi.p, oi.dtype, io + (j + 1) * oi.cstride, ld(oi.p, oi.dtype, io + j * oi.cstride));
            } else {
                st(ov.p, ov.dtype, vo + (j + 1) * ov.cstride, data);
                st(oi.p, oi.dtype, io + (j + 1) * oi.cstride, (float)c);
                break;
            }
        }
        if (j < 0) { st(ov.p, ov.dtype, vo, data); st(oi.p, oi.dtype, io, (float)c); }
    }
}

// RoPE, TensorApplyCPU.cs:1148-1178: one thread per (row, pair); trigonometry in double like the reference
__global__ void rope_rows_kernel(RowView r, RowView s, int seqLen, int rowOffset, double base) {
#pragma clang fp contract(off)
    long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const long half = s.cols / 2;
    if (idx >= s.rows * half) return;
    long row = idx / half; long i = idx % half;
    const long so = row_offset(s, row), ro = row_offset(r, row);
    int m = (int)(row % seqLen) + rowOffset;
    float theta = (float)pow(base, -2.0 * (double)i / (double)s.cols);
    float theta_m = theta * (float)m;
    float c = (float)cos((double)theta_m), sn = (float)sin((double)theta_m);
    float x0 = ld(s.p, s.dtype, so + (2 * i) * s.cstride), x1 = ld(s.p, s.dtype, so + (2 * i + 1) * s.cstride);
    st(r.p, r.dtype, ro + (2 * i) * r.cstride, x0 * c - x1 * sn);
    st(r.p, r.dtype, ro + (2 * i + 1) * r.cstride, x1 * c + x0 * sn);
}

// IndexSelect, TensorApplyCPU.cs:1306-1333: grid over (rows, col blocks)
__global__ void indexselect_kernel(RowView r, RowView s, const void* idx, int idt, long istride, int isAdd) {
    const long j = blockIdx.y; long c = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= r.cols) return;
    int src = (int)ld(idx, idt, j * istride);
    if (src < 0) return;
    float v = ld(s.p, s.dtype, row_offset(s, src) + c * s.cstride);
    long ro = row_offset(r, j) + c * r.cstride;
    st(r.p, r.dtype, ro, isAdd ? ld(r.p, r.dtype, ro) + v : v);
}
// IndexSelectGrad, TensorApplyCPU.cs:1336-1356: one thread per column walks the rows in order, so rows that hit the
// same destination are added in the reference's order
__global__ void indexselectgrad_kernel(RowView g, RowView a, const void* idx, int idt, long istride) {
    long c = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= a.cols) return;
    for (long j = 0; j < a.rows; ++j) {
        int dst = (int)ld(idx, idt, j * istride);
        if (dst < 0) continue;
        long go = row_offset(g, dst) + c * g.cstride;
        st(g.p, g.dtype, go, ld(g.p, g.dtype, go) + ld(a.p, a.dtype, row_offset(a, j) + c * a.cstride));
    }
}

__global__ void trimask_kernel(View r, long rows, long cols, float value, float masked, const void* lens, int ldt, int padded) {
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= rows * cols) return;
    long j = i / cols, id = i % cols;
    bool keep;
    if (!lens) keep = id <= j;                                   // BuildTriMask, TensorApplyCPU.cs:1016-1036
    else {                                                       // BuildSelfTriMask, TensorApplyCPU.cs:1040-1065
        long b = j / padded, sidx = j % padded;
        int ol = (int)ld(lens, ldt, b);
        keep = id < ol && sidx < ol && id <= sidx;
    }
    st(r.p, r.dtype, view_offset(r, i), keep ? value : masked);
}

__global__ void iscorrupted_kernel(View s, long n, int* flag) {
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float v = ld(s.p, s.dtype, view_offset(s, i));
    if (!isfinite(v)) *flag = 1;     // every writer stores the same value
}

static dim3 grid1(long n) { return dim3((unsigned)ceil_div(n, 256)); }
static void check_launch() { TSHIP_CHECK_HIP(hipGetLastError()); }

static void require_rows_match(const RowView& a, const RowView& b, const char* what) {
    if (a.rows != b.rows || a.cols != b.cols) throw Error(std::string(what) + ": result and source shapes differ");
}

}  // namespace tship

using namespace tship;

extern "C" {

TSHIP_API int TSHip_Copy(const TSHipTensor* result, const TSHipTensor* src) {
    TSHIP_BEGIN
    ensure_init();
    View r = make_view(result, "TSHip_Copy"), s = make_view(src, "TSHip_Copy");
    TSHIP_REQUIRE(count(r) == count(s), "TSHip_Copy: element counts differ");
    long n = count(r);
    if (n == 0) return 1;
    // the reference iterates each tensor in its own index order (TensorApplyCPU.cs:282-306)
    hipLaunchKernelGGL(ew_unary_kernel, grid1(n), dim3(256), 0, stream(), r, s, (int)EW_COPY, n);
    check_launch();
    TSHIP_END
}

TSHIP_API int TSHip_Fill(const TSHipTensor* result, float value) {
    TSHIP_BEGIN
    ensure_init();
    View r = make_view(result, "TSHip_Fill");
    long n = count(r);
    if (n == 0) return 1;
    hipLaunchKernelGGL(ew_fill_kernel, grid1(n), dim3(256), 0, stream(), r, value, n);
    check_launch();
    TSHIP_END
}

static void addmm_common(const char* what, const TSHipTensor* result, float beta, const TSHipTensor* src, float alpha, const TSHipTensor* m1,
                         const TSHipTensor* m2, int nd) {
    ensure_init();
    View r = make_view(result, what), s = make_view(src, what), a = make_view(m1, what), b = make_view(m2, what);
    // CpuBasicOps.Addmm / AddmmBatch argument checks (CpuBasicOps.cs:49-184)
    if (r.dtype != s.dtype || a.dtype != s.dtype || b.dtype != s.dtype) throw Error(std::string(what) + ": All tensors must have the same element type");
    if (s.nd != nd) throw Error(std::string(what) + ": src must be a matrix");
    if (a.nd != nd) throw Error(std::string(what) + ": m1 must be a matrix");
    if (b.nd != nd) throw Error(std::string(what) + ": m2 must be a matrix");
    if (r.nd != nd) throw Error(std::string(what) + ": result must be a matrix");
    const int o = nd - 2;
    if (s.sz[o] != a.sz[o] || s.sz[o + 1] != b.sz[o + 1] || a.sz[o + 1] != b.sz[o]) throw Error(std::string(what) + ": Size mismatch");
    if (!same_shape(r, s)) throw Error(std::string(what) + ": result has the wrong shape");
    long nb = 1;
    if (nd == 3) { nb = s.sz[0]; if (a.sz[0] != nb || b.sz[0] != nb) throw Error(std::string(what) + ": Size mismatch"); }
    const int M = (int)s.sz[o], N = (int)s.sz[o + 1], K = (int)a.sz[o + 1];
    if (M == 0 || N == 0 || nb == 0) return;
    auto mv = [&](const View& v) { MatView m; m.p = v.p; m.dtype = v.dtype; m.s0 = v.st[o]; m.s1 = v.st[o + 1]; m.sb = nd == 3 ? v.st[0] : 0; return m; };
    // fp16 operands with contiguous rows (Affine, Mul and AddmmBatch with an untransposed right operand): matrix cores
    const bool mfma = s.dtype == TSHIP_F16 && a.st[o + 1] == 1 && b.st[o + 1] == 1 && r.st[o + 1] == 1 && K % 8 == 0 && N % 4 == 0 && K >= 16 &&
                      a.st[o] % 8 == 0 && b.st[o] % 4 == 0 && ((uintptr_t)a.p % 16) == 0 && ((uintptr_t)b.p % 8) == 0 &&
                      (nd == 2 || (a.st[0] % 8 == 0 && b.st[0] % 4 == 0));
    if (mfma) {
        dim3 grid((unsigned)ceil_div(N, 64), (unsigned)ceil_div(M, 128), (unsigned)nb);
        hipLaunchKernelGGL(gemm_f16_mfma_kernel, grid, dim3(256), 0, stream(), mv(r), mv(s), mv(a), mv(b), M, N, K, alpha, beta);
    } else {
        dim3 grid((unsigned)ceil_div(N, 64), (unsigned)ceil_div(M, 64), (unsigned)nb);
        hipLaunchKernelGGL(gemm_strided_kernel, grid, dim3(256), 0, stream(), mv(r), mv(s), mv(a), mv(b), M, N, K, alpha, beta);
    }
    check_launch();
}

TSHIP_API int TSHip_Addmm(const TSHipTensor* result, float beta, const TSHipTensor* src, float alpha, const TSHipTensor* m1, const TSHipTensor* m2) {
    TSHIP_BEGIN
    addmm_common("TSHip_Addmm", result, beta, src, alpha, m1, m2, 2);
    TSHIP_END
}
TSHIP_API int TSHip_AddmmBatch(const TSHipTensor* result, float beta, const TSHipTensor* src, float alpha, const TSHipTensor* m1, const TSHipTensor* m2) {
    TSHIP_BEGIN
    addmm_common("TSHip_AddmmBatch", result, beta, src, alpha, m1, m2, 3);
    TSHIP_END
}

TSHIP_API int TSHip_IndexSelect(const TSHipTensor* result, const TSHipTensor* src, const TSHipTensor* indice, int is_add) {
    TSHIP_BEGIN
    ensure_init();
    View r = make_view(result, "TSHip_IndexSelect"), s = make_view(src, "TSHip_IndexSelect"), ix = make_view(indice, "TSHip_IndexSelect");
    TSHIP_REQUIRE(r.nd == 2 && s.nd == 2, "TSHip_IndexSelect: result and src must be matrices");
    TSHIP_REQUIRE(r.sz[1] == s.sz[1], "TSHip_IndexSelect: column counts differ");
    TSHIP_REQUIRE(count(ix) == r.sz[0], "TSHip_IndexSelect: one index per result row is required");
    RowView rr = row_view(r), sr = row_view(s);
    if (rr.rows == 0 || rr.cols == 0) return 1;
    // indices were validated against the source on neither side in the reference; here an out-of-range row would
    // fault the GPU, so the host checks them
    std::vector<float> hidx;
    {
        View c = ix; long n = count(ix);
        TSHIP_REQUIRE(is_contiguous(c) && c.dtype == TSHIP_F32, "TSHip_IndexSelect: indices must be a contiguous Float32 tensor");
        hidx.resize((size_t)n);
        TSHIP_CHECK_HIP(hipMemcpyAsync(hidx.data(), c.p, n * sizeof(float), hipMemcpyDeviceToHost, stream()));
        TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));
        for (float f : hidx) TSHIP_REQUIRE((int)f < s.sz[0], "TSHip_IndexSelect: index out of range");
    }
    dim3 grid((unsigned)ceil_div(rr.cols, 256), (unsigned)rr.rows);
    hipLaunchKernelGGL(indexselect_kernel, grid, dim3(256), 0, stream(), rr, sr, (const void*)ix.p, ix.dtype, 1L, is_add);
    check_launch();
    TSHIP_END
}

TSHIP_API int TSHip_IndexSelectGrad(const TSHipTensor* grad, const TSHipTensor* adj, const TSHipTensor* indice) {
    TSHIP_BEGIN
    ensure_init();
    View g = make_view(grad, "TSHip_IndexSelectGrad"), a = make_view(adj, "TSHip_IndexSelectGrad"), ix = make_view(indice, "TSHip_IndexSelectGrad");
    TSHIP_REQUIRE(g.nd == 2 && a.nd == 2, "TSHip_IndexSelectGrad: grad and adj must be matrices");
    TSHIP_REQUIRE(g.sz[1] == a.sz[1], "TSHip_IndexSelectGrad: column counts differ");
    TSHIP_REQUIRE(count(ix) == a.sz[0], "TSHip_IndexSelectGrad: one index per adj row is required");
    TSHIP_REQUIRE(is_contiguous(ix) && ix.dtype == TSHIP_F32, "TSHip_IndexSelectGrad: indices must be a contiguous Float32 tensor");
    long n = count(ix);
    if (n == 0 || a.sz[1] == 0) return 1;
    std::vector<float> hidx((size_t)n);
    TSHIP_CHECK_HIP(hipMemcpyAsync(hidx.data(), ix.p, n * sizeof(float), hipMemcpyDeviceToHost, stream()));
    TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));
    for (float f : hidx) TSHIP_REQUIRE((int)f < g.sz[0], "TSHip_IndexSelectGrad: index out of range");
    RowView gr = row_view(g), ar = row_view(a);
    hipLaunchKernelGGL(indexselectgrad_kernel, grid1(ar.cols), dim3(256), 0, stream(), gr, ar, (const void*)ix.p, ix.dtype, 1L);
    check_launch();
    TSHIP_END
}

static void rope_common(const TSHipTensor* result, const TSHipTensor* src, int seq_len, int row_offset, double base) {
    ensure_init();
    View r = make_view(result, "TSHip_RoPE"), s = make_view(src, "TSHip_RoPE");
    TSHIP_REQUIRE(same_shape(r, s), "TSHip_RoPE: result and src shapes differ");
    TSHIP_REQUIRE(seq_len >= 1, "TSHip_RoPE: seqLen must be positive");
    RowView rr = row_view(r), sr = row_view(s);
    TSHIP_REQUIRE(sr.cols % 2 == 0, "TSHip_RoPE: the last dimension must be even");
    long n = sr.rows * (sr.cols / 2);
    if (n == 0) return;
    hipLaunchKernelGGL(rope_rows_kernel, grid1(n), dim3(256), 0, stream(), rr, sr, seq_len, row_offset, base);
    check_launch();
}
TSHIP_API int TSHip_RoPE(const TSHipTensor* result, const TSHipTensor* src, int seq_len, int row_offset) {
    TSHIP_BEGIN
    rope_common(result, src, seq_len, row_offset, 500000.0);    // the reference's literal, TensorApplyCPU.cs:1161
    TSHIP_END
}
TSHIP_API int TSHip_RoPEEx(const TSHipTensor* result, const TSHipTensor* src, int seq_len, int row_offset, float base) {
    TSHIP_BEGIN
    rope_common(result, src, seq_len, row_offset, (double)base);
    TSHIP_END
}

static void norm_common(const char* what, const TSHipTensor* result, const TSHipTensor* src, const TSHipTensor* gamma, const TSHipTensor* beta, float eps, int layer) {
    ensure_init();
    View r = make_view(result, what), s = make_view(src, what), g = make_view(gamma, what);
    TSHIP_REQUIRE(same_shape(r, s), std::string(what) + ": result and src shapes differ");
    RowView rr = row_view(r), sr = row_view(s);
    TSHIP_REQUIRE(count(g) == sr.cols, std::string(what) + ": gamma must have one value per column");
    const void* bp = nullptr; int bdt = 0; long bs = 0;
    if (beta) {
        View b = make_view(beta, what);
        TSHIP_REQUIRE(count(b) == sr.cols, std::string(what) + ": beta must have one value per column");
        bp = b.p; bdt = b.dtype; bs = b.st[b.nd - 1];
    }
    if (sr.rows == 0 || sr.cols == 0) return;
    hipLaunchKernelGGL(norm_rows_kernel, dim3((unsigned)sr.rows), dim3(256), 0, stream(), rr, sr, (const void*)g.p, g.dtype, g.st[g.nd - 1], bp, bdt, bs, eps, layer);
    check_launch();
}
TSHIP_API int TSHip_RMSNorm(const TSHipTensor* result, const TSHipTensor* src, const TSHipTensor* gamma, const TSHipTensor* beta, float eps) {
    TSHIP_BEGIN
    norm_common("TSHip_RMSNorm", result, src, gamma, beta, eps, 0);
    TSHIP_END
}
TSHIP_API int TSHip_LayerNorm(const TSHipTensor* result, const TSHipTensor* src, const TSHipTensor* gamma, const TSHipTensor* beta, float eps) {
    TSHIP_BEGIN
    norm_common("TSHip_LayerNorm", result, src, gamma, beta, eps, 1);
    TSHIP_END
}

TSHIP_API int TSHip_Softmax(const TSHipTensor* result, const TSHipTensor* src) {
    TSHIP_BEGIN
    ensure_init();
    View r = make_view(result, "TSHip_Softmax"), s = make_view(src, "TSHip_Softmax");
    TSHIP_REQUIRE(same_shape(r, s), "TSHip_Softmax: result and src shapes differ");
    RowView rr = row_view(r), sr = row_view(s);
    if (sr.rows == 0 || sr.cols == 0) return 1;
    hipLaunchKernelGGL(softmax_rows_kernel, dim3((unsigned)sr.rows), dim3(256), 0, stream(), rr, sr);
    check_launch();
    TSHIP_END
}

TSHIP_API int TSHip_Argmax(const TSHipTensor* result, const TSHipTensor* src, int dim) {
    TSHIP_BEGIN
    ensure_init();
    View r = make_view(result, "TSHip_Argmax"), s = make_view(src, "TSHip_Argmax");
    TSHIP_REQUIRE(dim >= 0 && dim < s.nd, "TSHip_Argmax: dimension out of range");
    TSHIP_REQUIRE(r.nd == s.nd, "TSHip_Argmax: result must keep the reduced dimension with size 1");
    for (int i = 0; i < s.nd; ++i) TSHIP_REQUIRE(r.sz[i] == (i == dim ? 1 : s.sz[i]), "TSHip_Argmax: result has the wrong shape");
    // move `dim` last: a pure stride permutation
    View sp = s, rp = r;
    for (int i = dim; i < s.nd - 1; ++i) { std::swap(sp.sz[i], sp.sz[i + 1]); std::swap(sp.st[i], sp.st[i + 1]); std::swap(rp.sz[i], rp.sz[i + 1]); std::swap(rp.st[i], rp.st[i + 1]); }
    RowView rr = row_view(rp), sr = row_view(sp);
    TSHIP_REQUIRE(sr.cols >= 1, "TSHip_Argmax: empty dimension");
    if (sr.rows == 0) return 1;
    hipLaunchKernelGGL(argmax_rows_kernel, dim3((unsigned)sr.rows), dim3(256), 0, stream(), rr, sr);
    check_launch();
    TSHIP_END
}

TSHIP_API int TSHip_TopK(const TSHipTensor* out_val, const TSHipTensor* out_idx, const TSHipTensor* src, int k) {
    TSHIP_BEGIN
    ensure_init();
    View ov = make_view(out_val, "TSHip_TopK"), oi = make_view(out_idx, "TSHip_TopK"), s = make_view(src, "TSHip_TopK");
    RowView vr = row_view(ov), ir = row_view(oi), sr = row_view(s);
    TSHIP_REQUIRE(k >= 1 && k <= sr.cols, "TSHip_TopK: k out of range");
    TSHIP_REQUIRE(vr.cols == k && ir.cols == k && vr.rows == sr.rows && ir.rows == sr.rows, "TSHip_TopK: outputs must be [rows, k]");
    if (sr.rows == 0) return 1;
    hipLaunchKernelGGL(topk_rows_kernel, dim3((unsigned)ceil_div(sr.rows, 64)), dim3(64), 0, stream(), vr, ir, sr, k);
    check_launch();
    TSHIP_END
}

TSHIP_API int TSHip_BinaryTensor(int op, const TSHipTensor* result, const TSHipTensor* lhs, const TSHipTensor* rhs) {
    TSHIP_BEGIN
    ensure_init();
    TSHIP_REQUIRE(op >= TSHIP_ADD && op <= TSHIP_DIV, "TSHip_BinaryTensor: unknown op");
    View r = make_view(result, "TSHip_BinaryTensor"), a = make_view(lhs, "TSHip_BinaryTensor"), b = make_view(rhs, "TSHip_BinaryTensor");
    TSHIP_REQUIRE(same_shape(r, a) && same_shape(r, b), "TSHip_BinaryTensor: shapes differ (expand the operand first)");
    long n = count(r);
    if (n == 0) return 1;
    hipLaunchKernelGGL(ew_binary_kernel, grid1(n), dim3(256), 0, stream(), r, a, b, op, n);
    check_launch();
    TSHIP_END
}

TSHIP_API int TSHip_BinaryScalar(int op, const TSHipTensor* result, const TSHipTensor* src, float scalar) {
    TSHIP_BEGIN
    ensure_init();
    TSHIP_REQUIRE(op >= TSHIP_ADD && op <= TSHIP_DIV, "TSHip_BinaryScalar: unknown op");
    View r = make_view(result, "TSHip_BinaryScalar"), a = make_view(src, "TSHip_BinaryScalar");
    TSHIP_REQUIRE(same_shape(r, a), "TSHip_BinaryScalar: shapes differ");
    long n = count(r);
    if (n == 0) return 1;
    hipLaunchKernelGGL(ew_scalar_kernel, grid1(n), dim3(256), 0, stream(), r, a, scalar, op, n);
    check_launch();
    TSHIP_END
}

TSHIP_API int TSHip_Unary(int op, const TSHipTensor* result, const TSHipTensor* src) {
    TSHIP_BEGIN
    ensure_init();
    TSHIP_REQUIRE(op >= TSHIP_RELU && op <= TSHIP_ABS, "TSHip_Unary: unknown op");
    View r = make_view(result, "TSHip_Unary"), a = make_view(src, "TSHip_Unary");
    TSHIP_REQUIRE(same_shape(r, a), "TSHip_Unary: shapes differ");
    long n = count(r);
    if (n == 0) return 1;
    hipLaunchKernelGGL(ew_unary_kernel, grid1(n), dim3(256), 0, stream(), r, a, op, n);
    check_launch();
    TSHIP_END
}

TSHIP_API int TSHip_BuildTriMask(const TSHipTensor* result, float value, float masked_value) {
    TSHIP_BEGIN
    ensure_init();
    View r = make_view(result, "TSHip_BuildTriMask");
    TSHIP_REQUIRE(r.nd == 2, "TSHip_BuildTriMask: result must be a matrix");
    long n = count(r);
    if (n == 0) return 1;
    hipLaunchKernelGGL(trimask_kernel, grid1(n), dim3(256), 0, stream(), r, r.sz[0], r.sz[1], value, masked_value, (const void*)nullptr, 0, 1);
    check_launch();
    TSHIP_END
}

TSHIP_API int TSHip_BuildSelfTriMask(const TSHipTensor* result, const TSHipTensor* original_lengths, int padded_seq_len, float value, float masked_value) {
    TSHIP_BEGIN
    ensure_init();
    View r = make_view(result, "TSHip_BuildSelfTriMask"), l = make_view(original_lengths, "TSHip_BuildSelfTriMask");
    TSHIP_REQUIRE(r.nd == 2 && padded_seq_len >= 1, "TSHip_BuildSelfTriMask: result must be a matrix");
    TSHIP_REQUIRE(is_contiguous(l), "TSHip_BuildSelfTriMask: lengths must be contiguous");
    TSHIP_REQUIRE(count(l) * padded_seq_len >= r.sz[0], "TSHip_BuildSelfTriMask: one length per sequence is required");
    long n = count(r);
    if (n == 0) return 1;
    hipLaunchKernelGGL(trimask_kernel, grid1(n), dim3(256), 0, stream(), r, r.sz[0], r.sz[1], value, masked_value, (const void*)l.p, l.dtype, padded_seq_len);
    check_launch();
    TSHIP_END
}

// shared by gather and scatter_fill: a device flag for indices outside the dimension, read back after the kernel
static void run_indexed(const char* what, const std::function<void(int*)>& launch_fn) {
    int* flag = (int*)pool_alloc(sizeof(int));        // (a cached block after the first call: no driver call per pick of a beam loop)
    int host = 0;
    hipError_t e = hipMemsetAsync(flag, 0, sizeof(int), stream());
    if (e == hipSuccess) { launch_fn(flag); e = hipGetLastError(); }
    if (e == hipSuccess) e = hipMemcpyAsync(&host, flag, sizeof(int), hipMemcpyDeviceToHost, stream());
    if (e == hipSuccess) e = hipStreamSynchronize(stream());
    pool_release(flag);
    TSHIP_CHECK_HIP(e);
    if (host) throw Error(std::string(what) + ": an index lies outside the dimension");
}

TSHIP_API int TSHip_Gather(const TSHipTensor* result, const TSHipTensor* src, int dim, const TSHipTensor* indices) {
    TSHIP_BEGIN
    ensure_init();
    View r = make_view(result, "TSHip_Gather"), s = make_view(src, "TSHip_Gather"), ix = make_view(indices, "TSHip_Gather");
    // CpuIndexingOps.Gather, TensorSharp/Cpu/CpuIndexingOps.cs:23-56
    TSHIP_REQUIRE(r.nd == s.nd, "result and src must have same number of dimensions");
    TSHIP_REQUIRE(dim >= 0 && dim < r.nd, "TSHip_Gather: dim out of range");
    TSHIP_REQUIRE(ix.nd == s.nd, "src and indices must have same number of dimensions");
    TSHIP_REQUIRE(same_shape(r, ix), "result and indices must be the same size");
    for (int d = 0; d < r.nd; ++d) TSHIP_REQUIRE(d == dim || s.sz[d] == r.sz[d], "result and src must be the same size except in dimension dim");
    const long n = count(ix);
    if (n == 0) return 1;
    run_indexed("TSHip_Gather", [&](int* flag) { hipLaunchKernelGGL(gather_kernel, grid1(n), dim3(256), 0, stream(), r, s, ix, dim, n, flag); });
    TSHIP_END
}

TSHIP_API int TSHip_ScatterFill(const TSHipTensor* result, float value, int dim, const TSHipTensor* indices) {
    TSHIP_BEGIN
    ensure_init();
    View r = make_view(result, "TSHip_ScatterFill"), ix = make_view(indices, "TSHip_ScatterFill");
    // CpuIndexingOps.ScatterFill, TensorSharp/Cpu/CpuIndexingOps.cs:141-167
    TSHIP_REQUIRE(dim >= 0 && dim < r.nd, "TSHip_ScatterFill: dim out of range");
    TSHIP_REQUIRE(ix.nd == r.nd, "result and indices must have same number of dimensions");
    for (int d = 0; d < r.nd; ++d) TSHIP_REQUIRE(d == dim || ix.sz[d] == r.sz[d], "result and indices must be the same size except in dimension dim");
    const long n = count(ix);
    if (n == 0) return 1;
    run_indexed("TSHip_ScatterFill", [&](int* flag) { hipLaunchKernelGGL(scatter_fill_kernel, grid1(n), dim3(256), 0, stream(), r, ix, dim, value, n, flag); });
    TSHIP_END
}

TSHIP_API int TSHip_IsCorrupted(const TSHipTensor* src, int* corrupted) {
    TSHIP_BEGIN
    ensure_init();
    TSHIP_REQUIRE(corrupted != nullptr, "TSHip_IsCorrupted: output pointer is null");
    View s = make_view(src, "TSHip_IsCorrupted");
    long n = count(s);
    *corrupted = 0;
    if (n == 0) return 1;
    int* flag = (int*)pool_alloc(sizeof(int));
    hipError_t e = hipMemsetAsync(flag, 0, sizeof(int), stream());
    if (e == hipSuccess) { hipLaunchKernelGGL(iscorrupted_kernel, grid1(n), dim3(256), 0, stream(), s, n, flag); e = hipGetLastError(); }
    if (e == hipSuccess) e = hipMemcpyAsync(corrupted, flag, sizeof(int), hipMemcpyDeviceToHost, stream());
    if (e == hipSuccess) e = hipStreamSynchronize(stream());
    pool_release(flag);
    TSHIP_CHECK_HIP(e);
    TSHIP_END
}

static int topp_sample_op(const char* who, const TSHipTensor* result, const TSHipTensor* probs, const TSHipTensor* uniforms, float top_p,
                          float repeat_penalty, const int32_t* host_seqs, const int32_t* host_seq_lens, int seq_ld) {
    TSHIP_BEGIN
    ensure_init();
    View r = make_view(result, who), p = make_view(probs, who), u = make_view(uniforms, who);
    TSHIP_REQUIRE(p.nd == 2 && p.dtype == TSHIP_F32 && p.st[1] == 1, "TSHip_TopPSample: probs must be a Float32 matrix with contiguous rows");
    const long rows = p.sz[0], K = p.sz[1];
    TSHIP_REQUIRE(K >= 1 && K <= 262144, "TSHip_TopPSample: between 1 and 262144 columns are supported");
    TSHIP_REQUIRE(count(r) == rows && r.dtype == TSHIP_F32 && is_contiguous(r), "TSHip_TopPSample: result must be a contiguous Float32 [rows,1] tensor");
    TSHIP_REQUIRE(count(u) == rows && u.dtype == TSHIP_F32 && is_contiguous(u), "TSHip_TopPSample: uniforms must be a contiguous Float32 [rows] tensor");
    TSHIP_REQUIRE(std::isfinite(repeat_penalty), "TSHip_TopPSampleEx: the penalty must be finite");
    if (rows == 0) return 1;
    const bool decay = host_seqs != nullptr && repeat_penalty != 0.0f;
    if (decay) {
        TSHIP_REQUIRE(host_seq_lens && seq_ld >= 1, "TSHip_TopPSampleEx: sequences need their lengths and a row stride");
        for (long i = 0; i < rows; ++i) TSHIP_REQUIRE(host_seq_lens[i] >= 0 && host_seq_lens[i] <= seq_ld, "TSHip_TopPSampleEx: sequence length out of range");
    }
    const long last_ld = round_up(K, 64);
    const size_t sort_bytes = round_up((long)topp_scratch_bytes(rows, K), 256);
    const size_t last_bytes = decay ? (size_t)rows * last_ld * sizeof(int) : 0;
    const size_t seq_bytes = decay ? round_up((long)((size_t)rows * seq_ld * sizeof(int)), 256) : 0, len_bytes = decay ? round_up(rows * (long)sizeof(int), 256) : 0;
    char* scratch = (char*)pool_alloc(sort_bytes + last_bytes + seq_bytes + len_bytes);
    TopPArgs a; std::memset(&a, 0, sizeof(a));
    a.in = (const float*)p.p; a.ld = p.st[0]; a.V = (int)K; a.in_is_logits = 0; a.temperature = 1.0f;
    a.uniforms = (const float*)u.p; a.top_p = top_p;
    topp_carve(a, scratch, rows, K);
    a.out_f32 = (float*)r.p;
    hipError_t e = hipSuccess;
    if (decay) {
        // tokens outside [0, K) can never be candidates; the history kernel skips them
        int* last = (int*)(scratch + sort_bytes); int* d_seqs = (int*)(scratch + sort_bytes + last_bytes); int* d_lens = (int*)(scratch + sort_bytes + last_bytes + seq_bytes);
        e = hipMemsetAsync(last, 0xff, last_bytes, stream());
        if (e == hipSuccess) e = hipMemcpyAsync(d_seqs, host_seqs, (size_t)rows * seq_ld * sizeof(int), hipMemcpyHostToDevice, stream());
        if (e == hipSuccess) e = hipMemcpyAsync(d_lens, host_seq_lens, (size_t)rows * sizeof(int), hipMemcpyHostToDevice, stream());
        if (e == hipSuccess) {
            hipLaunchKernelGGL(history_kernel, dim3((unsigned)ceil_div(rows * (long)seq_ld, 256)), dim3(256), 0, stream(), (const int*)d_seqs, (int)rows, seq_ld, (long)seq_ld, 0,
                               (const int*)d_lens, (int)K, last, last_ld);
            e = hipGetLastError();
        }
        a.repeat_penalty = repeat_penalty; a.last_pos = last; a.last_ld = last_ld; a.row_lens = d_lens;
    }
    if (e == hipSuccess) {
        topp_run(a, (int)rows, [&](const char*, void (*kernel)(TopPArgs), dim3 grid, dim3 block, const TopPArgs& args) {
            hipLaunchKernelGGL(kernel, grid, block, 0, stream(), args);
        });
        e = hipGetLastError();
    }
    // (the host arrays must stay valid until the copies are done: synchronise before returning in every case)
    hipError_t es = hipStreamSynchronize(stream());
    if (e == hipSuccess) e = es;
    pool_release(scratch);
    TSHIP_CHECK_HIP(e);
    TSHIP_END
}

TSHIP_API int TSHip_TopPSample(const TSHipTensor* result, const TSHipTensor* probs, const TSHipTensor* uniforms, float top_p) {
    return topp_sample_op("TSHip_TopPSample", result, probs, uniforms, top_p, 0.0f, nullptr, nullptr, 0);
}

TSHIP_API int TSHip_TopPSampleNoAlloc(const TSHipTensor* result, const TSHipTensor* probs, const TSHipTensor* uniforms, float top_p) {
    TSHIP_BEGIN
    const int dev = current_device();
    TSHIP_REQUIRE(dev >= 0 && dev < NOALLOC_MAX_DEVICES && g_scratch_ptr[dev], "TSHip_TopPSampleNoAlloc: call TSHip_Init first (this entry point sets nothing up by itself)");
    const char* who = "TSHip_TopPSampleNoAlloc";
    View r = make_view(result, who), p = make_view(probs, who), u = make_view(uniforms, who);
    TSHIP_REQUIRE(p.nd == 2 && p.dtype == TSHIP_F32 && p.st[1] == 1, "TSHip_TopPSampleNoAlloc: probs must be a Float32 matrix with contiguous rows");
    const long rows = p.sz[0], K = p.sz[1];
    TSHIP_REQUIRE(K >= 1 && K <= 262144, "TSHip_TopPSampleNoAlloc: between 1 and 262144 columns are supported");
    TSHIP_REQUIRE(count(r) == rows && r.dtype == TSHIP_F32 && is_contiguous(r), "TSHip_TopPSampleNoAlloc: result must be a contiguous Float32 [rows,1] tensor");
    TSHIP_REQUIRE(count(u) == rows && u.dtype == TSHIP_F32 && is_contiguous(u), "TSHip_TopPSampleNoAlloc: uniforms must be a contiguous Float32 [rows] tensor");
    if (rows == 0) return 1;
    const size_t need = topp_scratch_bytes(rows, K);
    TSHIP_REQUIRE(need <= NOALLOC_SCRATCH_BYTES, "TSHip_TopPSampleNoAlloc: rows x columns needs " + std::to_string(need) + " bytes of scratch, the fixed scratch holds " +
                                                     std::to_string(NOALLOC_SCRATCH_BYTES) + " (about 300000 probabilities); use TSHip_TopPSample");
    TopPArgs a; std::memset(&a, 0, sizeof(a));
    a.in = (const float*)p.p; a.ld = p.st[0]; a.V = (int)K; a.in_is_logits = 0; a.temperature = 1.0f;
    a.uniforms = (const float*)u.p; a.top_p = top_p;
    // (every kernel of the pipeline writes what it later reads, digit counts included: nothing has to start at zero)
    topp_carve(a, g_scratch_ptr[dev], rows, K);
    a.out_f32 = (float*)r.p;
    topp_run(a, (int)rows, [&](const char*, void (*kernel)(TopPArgs), dim3 grid, dim3 block, const TopPArgs& args) {
        hipLaunchKernelGGL(kernel, grid, block, 0, stream(), args);
    });
    TSHIP_CHECK_HIP(hipGetLastError());
    TSHIP_END
}

TSHIP_API int TSHip_TopPSampleEx(const TSHipTensor* result, const TSHipTensor* probs, const TSHipTensor* uniforms, float top_p, float repeat_penalty,
                                 const int32_t* host_seqs, const int32_t* host_seq_lens, int seq_ld) {
    return topp_sample_op("TSHip_TopPSampleEx", result, probs, uniforms, top_p, repeat_penalty, host_seqs, host_seq_lens, seq_ld);
}

}  // extern "C"
