// ts_oracle.cpp — CPU restatement of the TensorSharp CPU backend and of the
// Seq2SeqSharp GPTDecoder op sequence, written from the reference's source text.
//
// THIS IS TEST INFRASTRUCTURE.  It is the checker the HIP path is compared with
// (tests, the smoke check, and the "cpu_baseline" leg of the benchmark).  Nothing
// in the product library links, loads or calls it.
//
// Everything is fp32, single precision accumulation in the reference's loop order
// (the reference CPU backend is fp32 only: TensorSharp/TensorApplyCPU.cs:24-34).
// Compile with -ffp-contract=off: the reference's managed loops do a separate
// multiply and add (System.Numerics.Vector<float> has no fused multiply-add).
//
// Pinning status of each function (what a test checks it against) is listed in
// oracle/README.md; functions whose behaviour is fixed by the reference's source
// text only say "parity unpinned" there.
//
// All paths below are relative to the reference checkout.

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>
#include <algorithm>
#include <functional>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_API extern "C" __attribute__((visibility("default")))

namespace orc {

static int g_threads = 1;          // 1 = the reference's own single-threaded loop order
static const int kVec = 8;         // Vector<float>.Count on an AVX2 host (hardware dependent in the reference)

// ---------------------------------------------------------------------------------------------
// Strided tensor views (TensorSharp/Tensor.cs:12-125, :295-440).  Strides are in elements.
// ---------------------------------------------------------------------------------------------
struct Tensor {
    std::shared_ptr<std::vector<float>> st;
    long off = 0;
    std::vector<long> sz, sd;

    Tensor() {}
    explicit Tensor(const std::vector<long>& sizes) : sz(sizes) {
        sd.resize(sz.size());
        long s = 1;
        for (int i = (int)sz.size() - 1; i >= 0; --i) { sd[i] = s; s *= sz[i]; }
        st = std::make_shared<std::vector<float>>((size_t)s, 0.0f);
    }
    static Tensor from(const float* p, const std::vector<long>& sizes) {
        Tensor t(sizes);
        std::memcpy(t.st->data(), p, sizeof(float) * t.count());
        return t;
    }
    bool defined() const { return (bool)st; }
    int nd() const { return (int)sz.size(); }
    long count() const { long c = 1; for (long v : sz) c *= v; return c; }
    float* p() const { return st->data() + off; }
    long rows() const { return sz[0]; }
    long cols() const { return sz[nd() - 1]; }

    // Tensor.IsContiguous (TensorSharp/Tensor.cs:254-268)
    bool contiguous() const {
        long s = 1;
        for (int i = nd() - 1; i >= 0; --i) {
            if (sd[i] != s) return false;
            s *= sz[i];
        }
        return true;
    }
    // Tensor.View (TensorSharp/Tensor.cs:295-312): only legal on contiguous tensors; -1 infers one dim
    Tensor view(std::vector<long> sizes) const {
        if (!contiguous()) throw std::runtime_error("Cannot use View on a non-contiguous tensor");
        long known = 1; int infer = -1;
        for (int i = 0; i < (int)sizes.size(); ++i) { if (sizes[i] == -1) infer = i; else known *= sizes[i]; }
        if (infer >= 0) sizes[infer] = count() / known;
        Tensor t; t.st = st; t.off = off; t.sz = sizes; t.sd.resize(sizes.size());
        long s = 1;
        for (int i = (int)sizes.size() - 1; i >= 0; --i) { t.sd[i] = s; s *= sizes[i]; }
        if (s != count()) throw std::runtime_error("Output tensor must have the same number of elements as the input");
        return t;
    }
    // Tensor.Transpose(d1,d2) (TensorSharp/Tensor.cs:380-400)
    Tensor transpose(int a, int b) const {
        Tensor t = *this; std::swap(t.sz[a], t.sz[b]); std::swap(t.sd[a], t.sd[b]); return t;
    }
    // Tensor.Expand (TensorSharp/Tensor.cs:415-440): size-1 dims get stride 0
    Tensor expand(const std::vector<long>& sizes) const {
        if ((int)sizes.size() != nd()) throw std::runtime_error("Expand: rank mismatch");
        Tensor t = *this;
        for (int i = 0; i < nd(); ++i) {
            if (sz[i] != sizes[i]) {
                if (sz[i] != 1) throw std::runtime_error("Can only expand singleton dimensions");
                t.sz[i] = sizes[i]; t.sd[i] = 0;
            }
        }
        return t;
    }
    // Tensor.Narrow (TensorSharp/Tensor.cs:330-352)
    Tensor narrow(int dim, long start, long len) const {
        Tensor t = *this; t.off += start * sd[dim]; t.sz[dim] = len; return t;
    }
    // Tensor.Select (TensorSharp/Tensor.cs:354-372): narrow to one index, drop the dim
    Tensor select(int dim, long idx) const {
        Tensor t = narrow(dim, idx, 1);
        t.sz.erase(t.sz.begin() + dim); t.sd.erase(t.sd.begin() + dim);
        return t;
    }
};

// TensorApplyCPU.Copy (TensorSharp/TensorApplyCPU.cs:282-306): element-wise strided copy.
static void copy(const Tensor& dst, const Tensor& src) {
    if (dst.count() != src.count()) throw std::runtime_error("copy: element count mismatch");
    int nd = src.nd();
    if (dst.sz != src.sz) throw std::runtime_error("copy: shape mismatch");
    long n = src.count();
    std::vector<long> idx(nd, 0);
    float* d = dst.p(); const float* s = src.p();
    bool dcont = dst.contiguous();
    long soff = 0, doff = 0;
    for (long e = 0; e < n; ++e) {
        d[dcont ? e : doff] = s[soff];
        for (int k = nd - 1; k >= 0; --k) {
            idx[k]++; soff += src.sd[k]; if (!dcont) doff += dst.sd[k];
            if (idx[k] < src.sz[k]) break;
            soff -= src.sd[k] * src.sz[k]; if (!dcont) doff -= dst.sd[k] * src.sz[k];
            idx[k] = 0;
        }
    }
}

// Ops.AsContiguous (TensorSharp/Ops.cs:24-34): same tensor if already contiguous, else a packed copy
static Tensor as_contiguous(const Tensor& t) {
    if (t.contiguous()) return t;
    Tensor r(t.sz);
    copy(r, t);
    return r;
}

// TensorConcatenation.Concat (TensorSharp/Core/TensorConcatenation.cs:9-45): new tensor, inputs copied in order
static Tensor concat(int dim, const std::vector<Tensor>& in) {
    std::vector<long> sz = in[0].sz;
    long tot = 0;
    for (auto& t : in) tot += t.sz[dim];
    sz[dim] = tot;
    Tensor r(sz);
    long at = 0;
    for (auto& t : in) {
        copy(r.narrow(dim, at, t.sz[dim]), t);
        at += t.sz[dim];
    }
    return r;
}

// ---------------------------------------------------------------------------------------------
// SGEMM (TensorSharp/Cpu/LinearAlgebra/SGEMM.cs), column-major netlib form, as driven by
// MatrixMultiplication.Gemm (TensorSharp/Cpu/MatrixMultiplication.cs:343-457).
// ---------------------------------------------------------------------------------------------

// SGEMM "N","N" branch, SGEMM.cs:482-549.  C (M x N, ld ldc) := alpha*A(M x K)*B(K x N) + beta*C.
// For every column J: scale C(:,J) by beta, then for L = 1..K: if B(L,J) != 0:
// TEMP = alpha*B(L,J); C(:,J) += TEMP*A(:,L).   One rounding for the product, one for the sum.
static void sgemm_nn(int M, int N, int K, float alpha, const float* A, int lda, const float* B, int ldb,
                     float beta, float* C, int ldc) {
    auto body = [&](int J, int i0, int i1) {
        float* c = C + (long)J * ldc;
        if (beta == 0.0f) { for (int i = i0; i < i1; ++i) c[i] = 0.0f; }
        else if (beta != 1.0f) { for (int i = i0; i < i1; ++i) c[i] *= beta; }
        const float* b = B + (long)J * ldb;
        for (int L = 0; L < K; ++L) {
            if (b[L] != 0.0f) {
                float temp = alpha * b[L];
                const float* a = A + (long)L * lda;
                for (int i = i0; i < i1; ++i) c[i] += temp * a[i];
            }
        }
    };
    if (g_threads <= 1) {
        for (int J = 0; J < N; ++J) body(J, 0, M);
    } else {
        // same per-element operation order; work split over (column, row-block) for wall time only
        const int blk = 512;
        int nb = (M + blk - 1) / blk;
#pragma omp parallel for collapse(2) schedule(static) num_threads(g_threads)
        for (int ib = 0; ib < nb; ++ib)
            for (int J = 0; J < N; ++J)
                body(J, ib * blk, std::min(M, ib * blk + blk));
    }
}

// SGEMM "T","N" branch, SGEMM.cs:565-608.  C(I,J) = alpha*dot(A(:,I),B(:,J)) + beta*C(I,J) where the dot is
// taken kVec elements at a time (Vector.Dot of one SIMD register, added to the running TEMP), the loop bound
// is "L <= K - vectorSize" (1-based), and the tail is scalar.
static float vec_dot(const float* a, const float* b) {
    float p[kVec];
    for (int i = 0; i < kVec; ++i) p[i] = a[i] * b[i];
    // horizontal add order of Vector.Dot is hardware dependent in the reference; pairwise is used here
    return ((p[0] + p[1]) + (p[2] + p[3])) + ((p[4] + p[5]) + (p[6] + p[7]));
}
static void sgemm_tn(int M, int N, int K, float alpha, const float* A, int lda, const float* B, int ldb,
                     float beta, float* C, int ldc) {
#pragma omp parallel for schedule(static) num_threads(g_threads) if (g_threads > 1)
    for (int J = 0; J < N; ++J) {
        for (int I = 0; I < M; ++I) {
            float temp = 0.0f;
            const float* a = A + (long)I * lda; const float* b = B + (long)J * ldb;
            int L = 0;
            for (; L + 1 <= K - kVec; L += kVec) temp += vec_dot(a + L, b + L);
            for (; L < K; ++L) temp += a[L] * b[L];
            float* c = C + I + (long)J * ldc;
            if (beta == 0.0f) *c = alpha * temp; else *c = alpha * temp + beta * (*c);
        }
    }
}

// MatrixMultiplication.Gemm (MatrixMultiplication.cs:343-457): choose the column-major formulation.
// a: [M,K], b: [K,N], c: [M,N], arbitrary 2-D strides.
static void gemm(float alpha, const Tensor& a, const Tensor& b, float beta, const Tensor& c) {
    if (a.sz[0] != c.sz[0] || b.sz[1] != c.sz[1] || a.sz[1] != b.sz[0]) throw std::runtime_error("Size mismatch");
    Tensor ac, bc, cc; bool copyC = false;
    if (c.sd[0] == 1 && c.sd[1] != 0 && c.sd[1] != 1) { ac = a; bc = b; cc = c; }
    else if (c.sd[1] == 1 && c.sd[0] != 0 && c.sd[0] != 1) {
        // row-major C: (a*b)' = b'*a'  — swap and transpose all three
        cc = c.transpose(0, 1); ac = b.transpose(0, 1); bc = a.transpose(0, 1);
    } else {
        Tensor cn(std::vector<long>{c.sz[1], c.sz[0]});
        cc = cn.transpose(0, 1); copy(cc, c); copyC = true; ac = a; bc = b;
    }
    auto norm = [](Tensor& t, bool& trans) {
        if (t.sd[0] == 1 && t.sd[1] != 0 && t.sd[1] != 1) trans = false;
        else if (t.sd[1] == 1 && t.sd[0] != 0 && t.sd[0] != 1) { trans = true; t = t.transpose(0, 1); }
        else {
            Tensor n(std::vector<long>{t.sz[1], t.sz[0]});
            Tensor n2 = n.transpose(0, 1); copy(n2, t); t = n2; trans = false;
        }
    };
    bool ta, tb; norm(ac, ta); norm(bc, tb);
    int m = (int)ac.sz[ta ? 1 : 0];
    int k = (int)bc.sz[tb ? 1 : 0];
    int n = (int)bc.sz[tb ? 0 : 1];
    int lda = (int)ac.sd[1], ldb = (int)bc.sd[1], ldc = (int)cc.sd[1];
    if (!ta && !tb) sgemm_nn(m, n, k, alpha, ac.p(), lda, bc.p(), ldb, beta, cc.p(), ldc);
    else if (ta && !tb) sgemm_tn(m, n, k, alpha, ac.p(), lda, bc.p(), ldb, beta, cc.p(), ldc);
    else {
        // "N","T" / "T","T" never arise on the decode path.  netlib's N,T loop has the same per-element order
        // as N,N (C(:,J) += alpha*B(J,L)*A(:,L) for L = 1..K), so B is packed column-major and N,N / T,N reused.
        Tensor bt = bc.transpose(0, 1);                       // logical [k,n]
        Tensor packed(std::vector<long>{bt.sz[1], bt.sz[0]});
        Tensor pv = packed.transpose(0, 1); copy(pv, bt);     // [k,n] with stride0 == 1
        if (!ta) sgemm_nn(m, n, k, alpha, ac.p(), lda, pv.p(), (int)pv.sd[1], beta, cc.p(), ldc);
        else sgemm_tn(m, n, k, alpha, ac.p(), lda, pv.p(), (int)pv.sd[1], beta, cc.p(), ldc);
    }
    if (copyC) copy(c, cc);
}

// CpuBasicOps.Addmm (TensorSharp/Cpu/CpuBasicOps.cs:49-114): result := src (unless same tensor), then
// result = alpha*m1*m2 + beta*result
static void addmm(const Tensor& result, float beta, const Tensor& src, float alpha, const Tensor& m1, const Tensor& m2) {
    if (src.sz[0] != m1.sz[0] || src.sz[1] != m2.sz[1] || m1.sz[1] != m2.sz[0]) throw std::runtime_error("Size mismatch");
    bool same = (result.st == src.st && result.off == src.off && result.sd == src.sd);
    if (!same) copy(result, src);
    gemm(alpha, m1, m2, beta, result);
}
// CpuBasicOps.AddmmBatch (CpuBasicOps.cs:116-184): per-batch Gemm loop (non-MKL branch)
static void addmmbatch(const Tensor& result, float beta, const Tensor& src, float alpha, const Tensor& m1, const Tensor& m2) {
    if (src.sz[1] != m1.sz[1] || src.sz[2] != m2.sz[2] || m1.sz[2] != m2.sz[1]) throw std::runtime_error("Size mismatch");
    bool same = (result.st == src.st && result.off == src.off && result.sd == src.sd);
    if (!same) copy(result, src);
    long nb = src.sz[0];
    int saved = g_threads;
    if (saved > 1 && nb >= saved) {
        // batches are independent: thread over them, each batch in the reference's serial order
        g_threads = 1;
#pragma omp parallel for schedule(static) num_threads(saved)
        for (long i = 0; i < nb; ++i) gemm(alpha, m1.select(0, i), m2.select(0, i), beta, result.select(0, i));
        g_threads = saved;
    } else {
        for (long i = 0; i < nb; ++i) gemm(alpha, m1.select(0, i), m2.select(0, i), beta, result.select(0, i));
    }
}

// ---------------------------------------------------------------------------------------------
// Row kernels of TensorSharp/TensorApplyCPU.cs.  All take packed [rows, cols] buffers, as the reference does
// (it takes the raw buffer start and rows = storageSize / cols, CpuBasicOps.cs:990-1123).
// ---------------------------------------------------------------------------------------------

// TensorApplyCPU.Softmax, TensorApplyCPU.cs:1230-1268
static void softmax(float* out, const float* in, long rows, long cols) {
#pragma omp parallel for schedule(static) num_threads(g_threads) if (g_threads > 1 && rows > 1)
    for (long j = 0; j < rows; ++j) {
        float* so = out + j * cols; const float* sp = in + j * cols;
        float mx = sp[0];
        for (long i = 1; i < cols; ++i) mx = std::max(mx, sp[i]);
        float sum = 0.0f;
        for (long i = 0; i < cols; ++i) {
            float ex = (float)std::exp((double)(sp[i] - mx));   // (float)Math.Exp(sp[i] - max)
            so[i] = ex; sum += ex;
        }
        for (long i = 0; i < cols; ++i) so[i] /= sum;
    }
}

// TensorApplyCPU.LayerNorm, TensorApplyCPU.cs:1360-1447.  Sum and squared sum are taken kVec lanes at a
// time with the reference's "i < cols - vectorSize" bound (the last full vector falls to the scalar tail).
static void layernorm(float* out, const float* in, const float* gamma, const float* beta, float eps, long rows, long cols) {
#pragma omp parallel for schedule(static) num_threads(g_threads) if (g_threads > 1 && rows > 1)
    for (long j = 0; j < rows; ++j) {
        float* so = out + j * cols; const float* sp = in + j * cols;
        float lane[kVec]; for (int q = 0; q < kVec; ++q) lane[q] = 0.0f;
        long i = 0;
        for (; i < cols - kVec; i += kVec) for (int q = 0; q < kVec; ++q) lane[q] += sp[i + q];
        float sum = ((lane[0] + lane[1]) + (lane[2] + lane[3])) + ((lane[4] + lane[5]) + (lane[6] + lane[7]));
        for (; i < cols; ++i) sum += sp[i];
        float mean = sum / (float)cols;
        float sq = 0.0f;
        for (i = 0; i < cols - kVec; i += kVec) {
            float e[kVec];
            for (int q = 0; q < kVec; ++q) { float d = sp[i + q] - mean; e[q] = d * d; }
            sq += ((e[0] + e[1]) + (e[2] + e[3])) + ((e[4] + e[5]) + (e[6] + e[7]));
        }
        for (; i < cols; ++i) { float d = sp[i] - mean; sq += d * d; }
        float sigma = (float)std::sqrt((double)(eps + sq / (float)cols));
        for (i = 0; i < cols; ++i) {
            float t = gamma[i] * ((sp[i] - mean) / sigma);
            if (beta) t += beta[i];
            so[i] = t;
        }
    }
}

// TensorApplyCPU.RMSNorm, TensorApplyCPU.cs:1451-1496
static void rmsnorm(float* out, const float* in, const float* gamma, const float* beta, float eps, long rows, long cols) {
    float N = (float)cols;
#pragma omp parallel for schedule(static) num_threads(g_threads) if (g_threads > 1 && rows > 1)
    for (long j = 0; j < rows; ++j) {
        float* y = out + j * cols; const float* x = in + j * cols;
        float sq = 0.0f;
        for (long i = 0; i < cols; ++i) sq += x[i] * x[i];
        float rms = (float)std::sqrt((double)(sq / N + eps));
        for (long i = 0; i < cols; ++i) {
            float b = beta ? beta[i] : 0.0f;
            y[i] = gamma[i] * (x[i] / rms) + b;
        }
    }
}

// TensorApplyCPU.RoPE, TensorApplyCPU.cs:1148-1178.  Base 500000 is a literal in the reference; it is a
// parameter here so that the device kernel's base argument can be exercised, and every parity run passes 500000.
static void rope(float* out, const float* in, long rows, long cols, int seqLen, int rowOffset, double base) {
#pragma omp parallel for schedule(static) num_threads(g_threads) if (g_threads > 1 && rows > 8)
    for (long j = 0; j < rows; ++j) {
        float* r = out + j * cols; const float* s = in + j * cols;
        int m = (int)(j % seqLen) + rowOffset;
        for (long id = 0; id < cols; ++id) {
            long i = id / 2;
            float theta = (float)std::pow(base, -2.0 * (double)i / (double)cols);
            float theta_m = theta * (float)m;
            float c = (float)std::cos((double)theta_m);
            float sn = (float)std::sin((double)theta_m);
            if (id % 2 == 0) r[id] = s[id] * c - s[id + 1] * sn;
            else r[id] = s[id] * c + s[id - 1] * sn;
        }
    }
}

// TensorApplyCPU.IndexSelect, TensorApplyCPU.cs:1306-1333 (indices are floats, negative rows are skipped)
static void indexselect(float* res, const float* src, const float* idx, long rows, long cols, bool isAdd) {
    for (long j = 0; j < rows; ++j) {
        int s = (int)idx[j];
        if (s >= 0) {
            float* r = res + j * cols; const float* q = src + (long)s * cols;
            for (long i = 0; i < cols; ++i) { if (!isAdd) r[i] = q[i]; else r[i] += q[i]; }
        }
    }
}
// TensorApplyCPU.IndexSelectGrad, TensorApplyCPU.cs:1336-1356 (used forward as IndexUpdate: scatter-add in row order)
static void indexselectgrad(float* grad, const float* adj, const float* idx, long rows, long cols) {
    for (long j = 0; j < rows; ++j) {
        int g = (int)idx[j];
        if (g >= 0) {
            const float* a = adj + j * cols; float* r = grad + (long)g * cols;
            for (long i = 0; i < cols; ++i) r[i] += a[i];
        }
    }
}

// TensorApplyCPU.replace_smaller / TopK, TensorApplyCPU.cs:1099-1146
static void replace_smaller(float* arr, float* arrIdx, int k, float data, float idx) {
    if (data < arr[k - 1]) return;
    for (int j = k - 2; j >= 0; --j) {
        if (data > arr[j]) { arr[j + 1] = arr[j]; arrIdx[j + 1] = arrIdx[j]; }
        else { arr[j + 1] = data; arrIdx[j + 1] = idx; return; }
    }
    arr[0] = data; arrIdx[0] = idx;
}
static void topk(float* outVal, float* outIdx, const float* in, int k, long rows, long cols) {
    for (long j = 0; j < rows; ++j) {
        float* ov = outVal + j * k; float* oi = outIdx + j * k; const float* r = in + j * cols;
        for (int i = 0; i < k; ++i) { ov[i] = -1.70141e+38f; oi[i] = -1.70141e+38f; }
        for (long i = 0; i < cols; ++i) replace_smaller(ov, oi, k, r[i], (float)i);
    }
}

// TensorApplyCPU.Argmax over the last dim, TensorApplyCPU.cs:339-360 (strict ">", first maximum wins)
static void argmax_lastdim(float* outIdx, const float* in, long rows, long cols) {
    for (long j = 0; j < rows; ++j) {
        const float* s = in + j * cols;
        float v = s[0]; float index = 0;
        for (long i = 1; i < cols; ++i) { if (s[i] > v) { v = s[i]; index = (float)i; } }
        outIdx[j] = index;
    }
}

// TensorApplyCPU.BuildTriMask, TensorApplyCPU.cs:1016-1036
static void buildtrimask(float* out, long rows, long cols, float value, float masked) {
    for (long j = 0; j < rows; ++j) for (long id = 0; id < cols; ++id) out[j * cols + id] = (id <= j) ? value : masked;
}
// TensorApplyCPU.BuildSelfTriMask, TensorApplyCPU.cs:1040-1065
static void buildselftrimask(float* out, const float* lens, long rows, long cols, int padded, float value, float masked) {
    for (long j = 0; j < rows; ++j) {
        int b = (int)(j / padded), s = (int)(j % padded);
        for (long id = 0; id < cols; ++id) {
            int ol = (int)lens[b];
            out[j * cols + id] = (id < ol && s < ol && id <= s) ? value : masked;
        }
    }
}

// activations, TensorApplyCPU.cs:1747-1801
static inline float relu(float w) { return w < 0.0f ? 0.0f : w; }
static inline float leakyrelu(float w) { return w < 0.0f ? 0.01f * w : w; }
static inline float silu(float w) { return w / (1.0f + (float)std::exp((double)(-w))); }

// TensorApplyCPU.IsCorrupted, TensorApplyCPU.cs:1212-1228
static bool iscorrupted(const float* p, long n) { for (long i = 0; i < n; ++i) if (!std::isfinite(p[i])) return true; return false; }

// float -> half, round to nearest even; overflow to infinity
// (ExternalProjects/managedCuda/ManagedCUDA/BasicTypesStructAsTypes.cs:800-840, :912-922)
static uint16_t float2half_bits(float f) {
    uint32_t x; std::memcpy(&x, &f, 4);
    uint32_t u = x & 0x7fffffffU, sign = (x >> 16) & 0x8000U, rem, res;
    if (u >= 0x7f800000U) { rem = 0; res = (u == 0x7f800000U) ? (sign | 0x7c00U) : 0x7fffU; }
    else if (u > 0x477fefffU) { rem = 0x80000000U; res = sign | 0x7bffU; }
    else if (u >= 0x38800000U) { rem = u << 19; u -= 0x38000000U; res = sign | (u >> 13); }
    else if (u < 0x33000001U) { rem = u; res = sign; }
    else {
        uint32_t e = u >> 23, shift = 0x7eU - e, man = (u & 0x7fffffU) | 0x800000U;
        rem = man << (32 - shift); res = sign | (man >> shift);
    }
    if (rem > 0x80000000U || (rem == 0x80000000U && (res & 1U))) res++;
    return (uint16_t)res;
}
static float half_bits2float(uint16_t h) {
    uint32_t s = (h & 0x8000U) << 16, e = (h >> 10) & 0x1f, m = h & 0x3ffU, x;
    if (e == 0) {
        if (m == 0) x = s;
        else { int sh = 0; while (!(m & 0x400U)) { m <<= 1; ++sh; } m &= 0x3ffU; x = s | ((uint32_t)(113 - sh) << 23) | (m << 13); }
    } else if (e == 31) x = s | 0x7f800000U | (m << 13);
    else x = s | ((e + 112) << 23) | (m << 13);
    float f; std::memcpy(&f, &x, 4); return f;
}

// ---------------------------------------------------------------------------------------------
// Graph-level ops (Seq2SeqSharp/Tools/ComputeGraphTensor.cs) at inference: allocate result, call the op.
// ---------------------------------------------------------------------------------------------
// g.Affine, ComputeGraphTensor.cs:1848-1880: Addmm(res, 1, bias.Expand(n,d), alpha=1, x, W)
static Tensor affine(const Tensor& x, const Tensor& W, const Tensor& b) {
    long n = x.sz[0], d = W.sz[1];
    Tensor res(std::vector<long>{n, d});
    addmm(res, 1.0f, b.expand({n, d}), 1.0f, x, W);
    return res;
}
// g.Mul(m1,m2), ComputeGraphTensor.cs:1752-1763: Addmm(res, 0, res, alpha, m1, m2)
static Tensor matmul(const Tensor& a, const Tensor& b) {
    Tensor res(std::vector<long>{a.sz[0], b.sz[1]});
    addmm(res, 0.0f, res, 1.0f, a, b);
    return res;
}
// g.MulBatch, ComputeGraphTensor.cs:1659-1666: AddmmBatch(res, 0, res, alpha, m1, m2)
static Tensor mulbatch(const Tensor& a, const Tensor& b, float alpha) {
    Tensor res(std::vector<long>{a.sz[0], a.sz[1], b.sz[2]});
    addmmbatch(res, 0.0f, res, alpha, a, b);
    return res;
}
static Tensor softmax_t(const Tensor& t) {   // g.Softmax, ComputeGraphTensor.cs:2444-2460 (rows = count/cols)
    Tensor c = as_contiguous(t); Tensor r(c.sz);
    softmax(r.p(), c.p(), c.count() / c.cols(), c.cols());
    return r;
}
static Tensor add_t(const Tensor& a, const Tensor& b) {   // g.Add, ComputeGraphTensor.cs:895-919; TensorApplyCPU.Add :378-408
    Tensor r(a.sz);
    Tensor bc = as_contiguous(b.sz == a.sz ? b : b.expand(a.sz)); Tensor ac = as_contiguous(a);
    long n = r.count(); float* rp = r.p(); const float* x = ac.p(); const float* y = bc.p();
    for (long i = 0; i < n; ++i) rp[i] = x[i] + y[i];
    return r;
}
static Tensor eltmul_t(const Tensor& a, const Tensor& b) {   // g.EltMul, ComputeGraphTensor.cs:826-833
    Tensor r(a.sz);
    Tensor bc = as_contiguous(b.sz == a.sz ? b : b.expand(a.sz)); Tensor ac = as_contiguous(a);
    long n = r.count(); float* rp = r.p(); const float* x = ac.p(); const float* y = bc.p();
    for (long i = 0; i < n; ++i) rp[i] = x[i] * y[i];
    return r;
}
static Tensor rope_t(const Tensor& t, int seqLen, int off, double base) {   // g.RoPE, ComputeGraphTensor.cs:490-497
    Tensor c = as_contiguous(t); Tensor r(c.sz);
    rope(r.p(), c.p(), c.count() / c.cols(), c.cols(), seqLen, off, base);
    return r;
}
static Tensor indexselect_t(const Tensor& src, const Tensor& idx) {   // g.IndexSelect, ComputeGraphTensor.cs:2791-2831
    Tensor s = as_contiguous(src);
    Tensor r(std::vector<long>{idx.sz[0], s.cols()});
    indexselect(r.p(), s.p(), idx.p(), r.sz[0], r.sz[1], false);
    return r;
}

// ---------------------------------------------------------------------------------------------
// Model (Seq2SeqSharp/Networks/GPTDecoder.cs + Layers/*), weights by the reference's saved names.
// ---------------------------------------------------------------------------------------------
struct Config {
    int n_layers, hidden, n_heads, n_kv_heads, ffn_dim, vocab;
    int attn_type;      // 0 = MultiHeadAttention (fused QKV), 1 = GroupQueryAttention
    int norm_type;      // 0 = RMSNorm, 1 = LayerNorm
    int act;            // 0 ReLU, 1 SiLU, 2 LeakyReLU, 3 "SwiGLU" as the reference computes it (gate without SiLU),
                        // 4 = gated with SiLU on the W1 branch (not a reference mode; for the device kernel's switch)
    int n_experts, experts_per_token;
    float norm_eps;
    float rope_base;    // the reference hard-codes 500000
    int use_rope;
    int max_segments;   // > 0: segment embeddings ("SegmentEmbedding" [max_segments, hidden], Utils/Misc.cs:164-168)
    int sep_token_id;   // vocabulary index of BuildInTokens.SEP
};

struct Model {
    Config c;
    std::map<std::string, Tensor> w;
    const Tensor& W(const std::string& n) const {
        auto it = w.find(n);
        if (it == w.end()) throw std::runtime_error("missing weight: " + n);
        return it->second;
    }
};

typedef std::map<std::string, Tensor> Cache;   // "{layer}_cached_K" / "_cached_V" (GPT.cs:236-247)

static Tensor norm(const Model& m, const std::string& prefix, const Tensor& x) {
    Tensor xc = as_contiguous(x); Tensor r(xc.sz);
    const Tensor& a = m.W(prefix + ".m_alpha");
    if (m.c.norm_type == 1) layernorm(r.p(), xc.p(), a.p(), m.W(prefix + ".m_beta").p(), m.c.norm_eps, xc.sz[0], xc.sz[1]);
    else rmsnorm(r.p(), xc.p(), a.p(), nullptr, m.c.norm_eps, xc.sz[0], xc.sz[1]);   // RMSNormalization.cs:33-37 passes beta = null
    return r;
}

static void act_inplace(int act, Tensor& t) {   // RunActivateFunction, PositionwiseFeedForward.cs:100-116
    float* p = t.p(); long n = t.count();
    if (act == 1 || act == 4) for (long i = 0; i < n; ++i) p[i] = silu(p[i]);
    else if (act == 0) for (long i = 0; i < n; ++i) p[i] = relu(p[i]);
    else if (act == 2) for (long i = 0; i < n; ++i) p[i] = leakyrelu(p[i]);
    // act == 3: nothing (the reference's SwiGLU applies no activation to the gate)
}

// shared tail of both attention layers: cache concat, scores, mask, softmax, AV, output projection, residual
static Tensor attn_tail(const Model& m, const std::string& name, Tensor Qs, Tensor Ks, Tensor Vs, const Tensor* mask,
                        long B, long Tq, long H, long d, const Tensor& inputQ, Cache* cache) {
    std::string kn = name + "_cached_K", vn = name + "_cached_V";
    if (cache) {
        auto ik = cache->find(kn);
        if (ik != cache->end()) Ks = concat(2, {ik->second, Ks});
        (*cache)[kn] = Ks;
        auto iv = cache->find(vn);
        if (iv != cache->end()) Vs = concat(1, {iv->second, Vs});
        (*cache)[vn] = Vs;
    }
    long Tkv = Ks.sz[2];
    float scale = 1.0f / (float)std::sqrt((double)d);
    Tensor attn = mulbatch(Qs, Ks, scale);                       // [B*H, Tq, Tkv]
    attn = attn.view({B, H, Tq, Tkv});
    if (mask) {                                                  // g.Add(attn, keyMask, inPlace)
        Tensor me = as_contiguous(*mask);
        float* a = attn.p(); const float* q = me.p(); long n = attn.count();
        for (long i = 0; i < n; ++i) a[i] = a[i] + q[i];
    }
    softmax(attn.p(), attn.p(), attn.count() / Tkv, Tkv);        // in place
    attn = attn.view({B * H, Tq, Tkv});
    Tensor o = mulbatch(attn, Vs, 1.0f).view({B, H, Tq, d});
    Tensor W = as_contiguous(o.transpose(1, 2)).view({B * Tq, H * d});
    Tensor fin = affine(W, m.W(name + ".W0"), m.W(name + ".b0"));
    return add_t(fin, inputQ);                                   // graph.Add(finalAttResults, inputQ)
}

// GroupQueryAttention.Perform, Seq2SeqSharp/Layers/GroupQueryAttention.cs:114-233
static Tensor gqa(const Model& m, int layer, const Tensor& inputQ, const Tensor* mask, long B, Cache* cache) {
    std::string name = "GPTDecoder.SelfAttn_" + std::to_string(layer);
    long H = m.c.n_heads, G = m.c.n_kv_heads, d = m.c.hidden / H, Tq = inputQ.sz[0] / B;
    Tensor n = norm(m, name + ".layerNormQ", inputQ);
    Tensor allQ = affine(n, m.W(name + ".Q"), m.W(name + ".Qb")).view({B, Tq, H, d});
    Tensor allK = affine(n, m.W(name + ".K"), m.W(name + ".Kb")).view({B, Tq, G, d});
    Tensor allV = affine(n, m.W(name + ".V"), m.W(name + ".Vb")).view({B, Tq, G, d});
    int ropeOffset = 0;
    if (cache) { auto it = cache->find(name + "_cached_K"); if (it != cache->end()) ropeOffset = (int)it->second.sz[2]; }
    Tensor Qs = as_contiguous(allQ.transpose(1, 2)).view({B * H, Tq, d});
    if (m.c.use_rope) Qs = rope_t(Qs, (int)Tq, ropeOffset, m.c.rope_base);
    long gs = H / G;
    Tensor Ks;
    if (m.c.use_rope) {
        Ks = as_contiguous(allK.transpose(1, 2)).view({B * G, Tq, d});
        Ks = rope_t(Ks, (int)Tq, ropeOffset, m.c.rope_base);
    } else Ks = as_contiguous(allK.transpose(1, 2));
    Ks = Ks.view({B, G, 1, Tq, d}).expand({B, G, gs, Tq, d}).transpose(3, 4);
    Ks = as_contiguous(Ks).view({B * H, d, Tq});
    Tensor Vs = as_contiguous(allV.transpose(1, 2));
    Vs = Vs.view({B, G, 1, Tq, d}).expand({B, G, gs, Tq, d});
    Vs = as_contiguous(Vs).view({B * H, Tq, d});
    return attn_tail(m, name, Qs, Ks, Vs, mask, B, Tq, H, d, inputQ, cache);
}

// MultiHeadAttention.PerformClassic, Seq2SeqSharp/Layers/MultiHeadAttention.cs:125-240
static Tensor mha(const Model& m, int layer, const Tensor& inputQ, const Tensor* mask, long B, Cache* cache) {
    std::string name = "GPTDecoder.SelfAttn_" + std::to_string(layer);
    long H = m.c.n_heads, d = m.c.hidden / H, Tq = inputQ.sz[0] / B;
    Tensor n = norm(m, name + ".layerNormQ", inputQ);
    Tensor qkv = affine(n, m.W(name + ".QKV"), m.W(name + ".QKVb")).view({B, Tq, 3, H, d});
    Tensor allQ = qkv.select(2, 0), allK = qkv.select(2, 1), allV = qkv.select(2, 2);
    int ropeOffset = 0;
    if (cache) { auto it = cache->find(name + "_cached_K"); if (it != cache->end()) ropeOffset = (int)it->second.sz[2]; }
    Tensor Qs = as_contiguous(allQ.transpose(1, 2)).view({B * H, Tq, d});
    if (m.c.use_rope) Qs = rope_t(Qs, (int)Tq, ropeOffset, m.c.rope_base);
    Tensor Ks;
    if (m.c.use_rope) {
        Ks = as_contiguous(allK.transpose(1, 2)).view({B * H, -1, d});
        Ks = rope_t(Ks, (int)Tq, ropeOffset, m.c.rope_base);
        Ks = as_contiguous(Ks.transpose(1, 2)).view({B * H, d, -1});
    } else Ks = as_contiguous(allK.transpose(1, 2).transpose(2, 3)).view({B * H, d, -1});
    Tensor Vs = as_contiguous(allV.transpose(1, 2)).view({B * H, -1, d});
    return attn_tail(m, name, Qs, Ks, Vs, mask, B, Tq, H, d, inputQ, cache);
}

// PositionwiseFeedForward.Process, Seq2SeqSharp/Layers/PositionwiseFeedForward.cs:72-98
static Tensor ffn(const Model& m, int layer, const Tensor& input) {
    std::string name = "GPTDecoder.PosFFN_" + std::to_string(layer);
    Tensor n = norm(m, name + ".layerNorm2", input);
    Tensor a = affine(n, m.W(name + ".feedForwardLayer1.m_Whd"), m.W(name + ".feedForwardLayer1.m_Bd"));
    act_inplace(m.c.act, a);
    if (m.c.act == 3 || m.c.act == 4) {
        Tensor c = affine(n, m.W(name + ".feedForwardLayer3.m_Whd"), m.W(name + ".feedForwardLayer3.m_Bd"));
        a = eltmul_t(a, c);
    }
    Tensor y = affine(a, m.W(name + ".feedForwardLayer2.m_Whd"), m.W(name + ".feedForwardLayer2.m_Bd"));
    return add_t(y, input);
}

// MoEFeedForward.Process, Seq2SeqSharp/Layers/MoEFeedForward.cs:76-181.  Optional outputs expose the routing
// (top-k indices per token, expert-major token lists) so that index parity can be checked bit for bit.
struct MoETrace { std::vector<float> topIdx, topVal, probs; std::vector<std::vector<float>> lists; };
static Tensor moe(const Model& m, int layer, const Tensor& input, MoETrace* trace) {
    std::string name = "GPTDecoder.MoEFFN_" + std::to_string(layer);
    int E = m.c.n_experts, k = m.c.experts_per_token;
    Tensor xc = as_contiguous(input); Tensor n(xc.sz);
    layernorm(n.p(), xc.p(), m.W(name + ".layerNorm.m_alpha").p(), m.W(name + ".layerNorm.m_beta").p(), m.c.norm_eps, xc.sz[0], xc.sz[1]);
    Tensor r = affine(n, m.W(name + ".m_Router"), m.W(name + ".m_RouterBias"));       // [R,E]
    Tensor maskT(std::vector<long>{1, (long)E});
    for (int i = 0; i < E; ++i) maskT.p()[i] = -65000.0f;                              // Dropout is a no-op at inference
    r = add_t(r, maskT.expand(r.sz));
    Tensor p = softmax_t(r);
    long R = input.sz[0];
    std::vector<float> tv((size_t)R * k), ti((size_t)R * k);
    topk(tv.data(), ti.data(), p.p(), k, R, E);
    std::vector<std::vector<float>> lists(E);
    for (long i = 0; i < R; ++i) for (int j = 0; j < k; ++j) lists[(int)ti[i * k + j]].push_back((float)i);
    if (trace) { trace->topIdx = ti; trace->topVal = tv; trace->lists = lists; trace->probs.assign(p.p(), p.p() + p.count()); }
    std::vector<Tensor> embs, idxs;
    const Tensor& W1 = m.W(name + ".m_Whd1"); const Tensor& W2 = m.W(name + ".m_Whd2");
    for (int e = 0; e < E; ++e) {
        if (lists[e].empty()) continue;
        Tensor sc = as_contiguous(p.narrow(1, e, 1));                                   // Peek(inputRouter,1,e) made contiguous
        Tensor idx = Tensor::from(lists[e].data(), {(long)lists[e].size(), 1});
        Tensor tvE = indexselect_t(sc, idx).expand({(long)lists[e].size(), n.sz[1]});
        Tensor t = indexselect_t(n, idx);
        t = matmul(t, W1.select(0, e));
        act_inplace(m.c.act, t);
        t = matmul(t, W2.select(0, e));
        t = eltmul_t(t, tvE);
        embs.push_back(t); idxs.push_back(idx);
    }
    Tensor all = concat(0, embs), allIdx = concat(0, idxs);
    Tensor res(n.sz);                                                                   // cleared
    indexselectgrad(res.p(), all.p(), allIdx.p(), all.sz[0], all.sz[1]);
    return add_t(input, res);
}

// GPTDecoder.Decode, Seq2SeqSharp/Networks/GPTDecoder.cs:153-191
static Tensor decoder(const Model& m, Tensor x, const Tensor* mask, long B, Cache* cache, std::vector<MoETrace>* traces) {
    Tensor maskE;
    if (mask) maskE = mask->expand({B, (long)m.c.n_heads, mask->sz[2], mask->sz[3]});
    for (int k = 0; k < m.c.n_layers; ++k) {
        Tensor x2 = (m.c.attn_type == 1) ? gqa(m, k, x, mask ? &maskE : nullptr, B, cache)
                                         : mha(m, k, x, mask ? &maskE : nullptr, B, cache);
        if (m.c.n_experts > 1 && k > 1) {
            MoETrace tr; x = moe(m, k, x2, traces ? &tr : nullptr);
            if (traces) traces->push_back(tr);
        } else x = ffn(m, k, x2);
    }
    return norm(m, "GPTDecoder.layerNorm", x);
}

// Decoder.GPTDecode (inference branch), Seq2SeqSharp/Applications/Decoder.cs:648-794, up to the probabilities.
// seqs: B rows of `len` token ids (the whole sequence so far).  With a non-empty cache only the last token
// of each row is fed (Decoder.cs:661-678); otherwise the whole sequence with a causal mask (:679-700).
// Returns probs [B,V]; logits (before softmax, after the temperature division) are written to logitsOut if given.
// lens (optional): the sequences' lengths before PadSentences made them `len` long (Decoder.cs:656); given, the mask of the
// full-sequence branch is BuildSelfTriMask over them (Decoder.cs:687-690, PaddingType other than NoPadding, batch > 1).
static Tensor gpt_step(const Model& m, const int* seqs, long B, long len, Cache* cache, float temperature, bool sampling,
                       float* logitsOut, std::vector<MoETrace>* traces, float* hiddenOut, const float* lens = nullptr) {
    long Tq; std::vector<float> ids;
    Tensor mask; bool haveMask = false;
    if (cache && !cache->empty()) {
        Tq = 1; ids.resize(B);
        for (long b = 0; b < B; ++b) ids[b] = (float)seqs[b * len + len - 1];
    } else {
        Tq = len; ids.resize(B * len);
        for (long i = 0; i < B * len; ++i) ids[i] = (float)seqs[i];
        if (lens) {
            mask = Tensor(std::vector<long>{B, Tq, Tq});
            buildselftrimask(mask.p(), lens, B * Tq, Tq, (int)Tq, 0.0f, -30000.0f);     // g.BuildSelfTriMask, ComputeGraphTensor.cs:3903-3909
            mask = mask.view({B, 1, Tq, Tq}); haveMask = true;
        } else {
            mask = Tensor(std::vector<long>{Tq, Tq});
            buildtrimask(mask.p(), Tq, Tq, 0.0f, -30000.0f);                            // g.BuildTriMask, ComputeGraphTensor.cs:3932-3935
            mask = mask.view({1, 1, Tq, Tq}); haveMask = true;
        }
    }
    // TensorUtils.CreateTokensEmbeddings, Utils/TensorUtils.cs:44-162: IndexSelect then Mul(scalar) in place
    const Tensor& E = m.W("TgtEmbeddings");
    Tensor idx = Tensor::from(ids.data(), {(long)ids.size(), 1});
    Tensor x = indexselect_t(E, idx);
    float scale = (float)std::sqrt((double)E.sz[1]);
    if (scale != 1.0f) { float* p = x.p(); long n = x.count(); for (long i = 0; i < n; ++i) p[i] = p[i] * scale; }
    if (m.c.max_segments > 0) {
        // TensorUtils.cs:60-72, 147-152: the segment index of a token is the number of SEP tokens before it in the list that is
        // fed (the whole sequence, or only its last token on a cached step: then always 0); embeddingRst = Add(embeddingRst,
        // IndexSelect(segmentEmbedding, segIdxs))
        std::vector<float> seg(ids.size());
        for (long b = 0; b < B; ++b) {
            int s_idx = 0;
            for (long j = 0; j < Tq; ++j) {
                seg[b * Tq + j] = (float)s_idx;
                if ((int)ids[b * Tq + j] == m.c.sep_token_id) ++s_idx;
            }
        }
        Tensor sx = indexselect_t(m.W("SegmentEmbedding"), Tensor::from(seg.data(), {(long)seg.size(), 1}));
        float* p = x.p(); const float* q = sx.p(); long n = x.count();
        for (long i = 0; i < n; ++i) p[i] = p[i] + q[i];
    }
    Tensor out = decoder(m, x, haveMask ? &mask : nullptr, B, cache, traces);
    std::vector<float> last(B);
    for (long i = 0; i < B; ++i) last[i] = (float)(Tq * (i + 1) - 1);
    out = indexselect_t(out, Tensor::from(last.data(), {B, 1}));
    if (hiddenOut) std::memcpy(hiddenOut, out.p(), sizeof(float) * out.count());
    Tensor logits = affine(out, m.W("FeedForward_Decoder_0.m_Whd"), m.W("FeedForward_Decoder_0.m_Bd"));
    if (sampling && temperature != 1.0f) { float* p = logits.p(); long n = logits.count(); for (long i = 0; i < n; ++i) p[i] = p[i] / temperature; }
    if (logitsOut) std::memcpy(logitsOut, logits.p(), sizeof(float) * logits.count());
    softmax(logits.p(), logits.p(), B, logits.sz[1]);                                   // in place
    return logits;
}

// g.TopPSample, Seq2SeqSharp/Tools/ComputeGraphTensor.cs:2305-2403.  `uniforms[i]` replaces the reference's
// RandomGenerator.floatRandom(0,1) draw for row i (one draw per row, rows in order).
static void toppsample(float* out, const float* probs, long rows, long K, float topP, float repeatPenalty,
                       const int* seqs, long seqLen, const float* uniforms) {
    for (long i = 0; i < rows; ++i) {
        std::map<int, int> dist;
        if (seqs) for (long j = 0; j < seqLen; ++j) dist[seqs[i * seqLen + j]] = (int)(seqLen - j);
        std::map<float, std::vector<int>> groups;          // SortedDictionary<float, List<int>>
        for (long j = 0; j < K; ++j) {
            float w = probs[i * K + j];
            if (w <= 0.0f) continue;
            auto it = dist.find((int)j);
            if (it != dist.end()) {
                float rp = (float)std::pow((double)((float)it->second / (float)seqLen), (double)repeatPenalty);
                w = (float)(w * rp);
            }
            groups[w].push_back((int)j);
        }
        float acc = 0.0f; std::vector<int> cands; std::vector<float> accP;
        for (auto it = groups.rbegin(); it != groups.rend(); ++it) {
            for (int id : it->second) {
                acc += it->first; cands.push_back(id); accP.push_back(acc);
                if (acc >= topP) break;
            }
            if (acc >= topP) break;
        }
        float u = uniforms[i];
        out[i] = 0.0f;
        for (size_t k = 0; k < accP.size(); ++k) if (accP[k] / acc >= u) { out[i] = (float)cands[k]; break; }
    }
}

}  // namespace orc

// =============================================================================================
// C entry points for ctypes
// =============================================================================================
using namespace orc;

static thread_local std::string g_err;
#define ORC_TRY try {
#define ORC_CATCH } catch (const std::exception& e) { g_err = e.what(); return 0; } return 1;

ORC_API const char* orc_last_error() { return g_err.c_str(); }
ORC_API void orc_set_threads(int n) {
#ifdef _OPENMP
    g_threads = n < 1 ? 1 : n;
#else
    (void)n; g_threads = 1;
#endif
}
ORC_API int orc_get_threads() { return g_threads; }

static Tensor wrap2(const float* p, long r, long c, long s0, long s1) {
    // copy into an owned buffer that spans the view, keep the strides
    long span = (r - 1) * std::abs(s0) + (c - 1) * std::abs(s1) + 1;
    Tensor t; t.st = std::make_shared<std::vector<float>>(p, p + span); t.off = 0; t.sz = {r, c}; t.sd = {s0, s1};
    return t;
}

// result[M,N] (contiguous, in/out) = alpha * m1 * m2 + beta * src ; src given with strides (stride 0 = broadcast)
ORC_API int orc_addmm(float* result, float beta, const float* src, long src_s0, long src_s1, float alpha,
                      const float* m1, long m1_s0, long m1_s1, const float* m2, long m2_s0, long m2_s1, long M, long K, long N) {
    ORC_TRY
    Tensor r(std::vector<long>{M, N});
    Tensor s = wrap2(src, M, N, src_s0, src_s1);
    Tensor a = wrap2(m1, M, K, m1_s0, m1_s1), b = wrap2(m2, K, N, m2_s0, m2_s1);
    addmm(r, beta, s, alpha, a, b);
    std::memcpy(result, r.p(), sizeof(float) * M * N);
    ORC_CATCH
}
ORC_API int orc_addmmbatch(float* result, float beta, const float* src, float alpha, const float* m1, const float* m2,
                           long nb, long M, long K, long N, int m2_transposed) {
    ORC_TRY
    Tensor r(std::vector<long>{nb, M, N});
    Tensor s = Tensor::from(src, {nb, M, N});
    Tensor a = Tensor::from(m1, {nb, M, K});
    Tensor b = m2_transposed ? Tensor::from(m2, {nb, N, K}).transpose(1, 2) : Tensor::from(m2, {nb, K, N});
    addmmbatch(r, beta, s, alpha, a, b);
    std::memcpy(result, r.p(), sizeof(float) * nb * M * N);
    ORC_CATCH
}
ORC_API void orc_softmax(float* out, const float* in, long rows, long cols) { softmax(out, in, rows, cols); }
ORC_API void orc_layernorm(float* out, const float* in, const float* g, const float* b, float eps, long rows, long cols) { layernorm(out, in, g, b, eps, rows, cols); }
ORC_API void orc_rmsnorm(float* out, const float* in, const float* g, const float* b, float eps, long rows, long cols) { rmsnorm(out, in, g, b, eps, rows, cols); }
ORC_API void orc_rope(float* out, const float* in, long rows, long cols, int seqLen, int rowOffset, double base) { rope(out, in, rows, cols, seqLen, rowOffset, base); }
ORC_API void orc_indexselect(float* res, const float* src, const float* idx, long rows, long cols, int isAdd) { indexselect(res, src, idx, rows, cols, isAdd != 0); }
ORC_API void orc_indexselectgrad(float* grad, const float* adj, const float* idx, long rows, long cols) { indexselectgrad(grad, adj, idx, rows, cols); }
ORC_API void orc_topk(float* ov, float* oi, const float* in, int k, long rows, long cols) { topk(ov, oi, in, k, rows, cols); }
ORC_API void orc_argmax(float* oi, const float* in, long rows, long cols) { argmax_lastdim(oi, in, rows, cols); }
ORC_API void orc_buildtrimask(float* out, long rows, long cols, float v, float mv) { buildtrimask(out, rows, cols, v, mv); }
ORC_API void orc_buildselftrimask(float* out, const float* lens, long rows, long cols, int padded, float v, float mv) { buildselftrimask(out, lens, rows, cols, padded, v, mv); }
ORC_API void orc_unary(int op, float* out, const float* in, long n) {
    for (long i = 0; i < n; ++i) out[i] = op == 0 ? relu(in[i]) : op == 1 ? silu(in[i]) : leakyrelu(in[i]);
}
ORC_API int orc_iscorrupted(const float* p, long n) { return iscorrupted(p, n) ? 1 : 0; }
ORC_API void orc_float2half(uint16_t* out, const float* in, long n) { for (long i = 0; i < n; ++i) out[i] = float2half_bits(in[i]); }
ORC_API void orc_half2float(float* out, const uint16_t* in, long n) { for (long i = 0; i < n; ++i) out[i] = half_bits2float(in[i]); }
ORC_API void orc_toppsample(float* out, const float* probs, long rows, long K, float topP, float repeatPenalty,
                            const int* seqs, long seqLen, const float* uniforms) {
    toppsample(out, probs, rows, K, topP, repeatPenalty, seqs, seqLen, uniforms);
}
// strided copy of a <=5-D view into a packed buffer (Ops.AsContiguous)
ORC_API int orc_copy_strided(float* dst, const float* src, long src_span, int nd, const long* sizes, const long* strides) {
    ORC_TRY
    Tensor s; s.st = std::make_shared<std::vector<float>>(src, src + src_span); s.off = 0;
    s.sz.assign(sizes, sizes + nd); s.sd.assign(strides, strides + nd);
    Tensor r(s.sz); copy(r, s);
    std::memcpy(dst, r.p(), sizeof(float) * r.count());
    ORC_CATCH
}

// ---- model -------------------------------------------------------------------------------
struct OrcGpt { Model m; Cache cache; std::vector<MoETrace> traces; };

ORC_API void* orc_gpt_create(const Config* c) { auto* g = new OrcGpt(); g->m.c = *c; return g; }
ORC_API void orc_gpt_destroy(void* h) { delete (OrcGpt*)h; }
ORC_API int orc_gpt_set_weight(void* h, const char* name, const float* data, int nd, const long* sizes) {
    ORC_TRY
    ((OrcGpt*)h)->m.w[name] = Tensor::from(data, std::vector<long>(sizes, sizes + nd));
    ORC_CATCH
}
ORC_API void orc_gpt_reset_cache(void* h) { ((OrcGpt*)h)->cache.clear(); }
ORC_API long orc_gpt_cache_len(void* h) {
    auto* g = (OrcGpt*)h; auto it = g->cache.find("GPTDecoder.SelfAttn_0_cached_K");
    return it == g->cache.end() ? 0 : it->second.sz[2];
}
// One GPTDecode call.  use_cache = 0 reproduces UseKVCache=false (full recompute, Decoder.cs:679-700).
// probs_out [B,V]; logits_out, hidden_out optional.
ORC_API int orc_gpt_step(void* h, const int* seqs, long B, long len, int use_cache, float temperature, int sampling,
                         float* probs_out, float* logits_out, float* hidden_out) {
    ORC_TRY
    auto* g = (OrcGpt*)h;
    g->traces.clear();
    Tensor p = gpt_step(g->m, seqs, B, len, use_cache ? &g->cache : nullptr, temperature, sampling != 0, logits_out, &g->traces, hidden_out);
    if (probs_out) std::memcpy(probs_out, p.p(), sizeof(float) * p.count());
    ORC_CATCH
}
// The same call on sequences that PadSentences brought to one length: seqs [B, len] padded (with the END tag), lens [B]
// their original lengths as floats (BuildInTokens.PadSentences returns them so).
ORC_API int orc_gpt_step_padded(void* h, const int* seqs, long B, long len, const float* lens, int use_cache, float temperature, int sampling,
                                float* probs_out, float* logits_out, float* hidden_out) {
    ORC_TRY
    auto* g = (OrcGpt*)h;
    g->traces.clear();
    Tensor p = gpt_step(g->m, seqs, B, len, use_cache ? &g->cache : nullptr, temperature, sampling != 0, logits_out, &g->traces, hidden_out, lens);
    if (probs_out) std::memcpy(probs_out, p.p(), sizeof(float) * p.count());
    ORC_CATCH
}
// copy a cache tensor out: which = 0 K ([B*H, d, T]), 1 V ([B*H, T, d]); returns element count (0 if absent)
ORC_API long orc_gpt_get_cache(void* h, int layer, int which, float* out, long cap) {
    auto* g = (OrcGpt*)h;
    std::string n = "GPTDecoder.SelfAttn_" + std::to_string(layer) + (which ? "_cached_V" : "_cached_K");
    auto it = g->cache.find(n); if (it == g->cache.end()) return 0;
    Tensor c = as_contiguous(it->second); long cnt = c.count();
    if (out && cap >= cnt) std::memcpy(out, c.p(), sizeof(float) * cnt);
    return cnt;
}
// install a cache tensor (for timing decode steps at a given context length without running the prefill)
ORC_API int orc_gpt_set_cache(void* h, int layer, int which, const float* data, long BH, long T, long d) {
    ORC_TRY
    auto* g = (OrcGpt*)h;
    std::string n = "GPTDecoder.SelfAttn_" + std::to_string(layer) + (which ? "_cached_V" : "_cached_K");
    g->cache[n] = which ? Tensor::from(data, {BH, T, d}) : Tensor::from(data, {BH, d, T});
    ORC_CATCH
}
// routing of MoE layer number `moe_ordinal` (0 = first MoE layer) from the last step
ORC_API long orc_gpt_moe_trace(void* h, int moe_ordinal, float* top_idx, float* top_val, float* probs, long cap) {
    auto* g = (OrcGpt*)h;
    if (moe_ordinal < 0 || moe_ordinal >= (int)g->traces.size()) return -1;
    auto& t = g->traces[moe_ordinal]; long n = (long)t.topIdx.size();
    if (cap >= n) {
        if (top_idx) std::memcpy(top_idx, t.topIdx.data(), sizeof(float) * n);
        if (top_val) std::memcpy(top_val, t.topVal.data(), sizeof(float) * n);
    }
    if (probs) std::memcpy(probs, t.probs.data(), sizeof(float) * t.probs.size());
    return n;
}
// a single MoE layer on its own: x [R,h] -> y [R,h], routing written out (expert-major token lists flattened)
ORC_API int orc_moe_layer(void* h, int layer, const float* x, long R, float* y, float* top_idx, float* top_val, float* probs) {
    ORC_TRY
    auto* g = (OrcGpt*)h;
    MoETrace tr;
    Tensor in = Tensor::from(x, {R, (long)g->m.c.hidden});
    Tensor out = moe(g->m, layer, in, &tr);
    std::memcpy(y, out.p(), sizeof(float) * out.count());
    if (top_idx) std::memcpy(top_idx, tr.topIdx.data(), sizeof(float) * tr.topIdx.size());
    if (top_val) std::memcpy(top_val, tr.topVal.data(), sizeof(float) * tr.topVal.size());
    if (probs) std::memcpy(probs, tr.probs.data(), sizeof(float) * tr.probs.size());
    ORC_CATCH
}
// single layers on their own (for per-op replay tests): attention with an optional causal mask and the model's cache
ORC_API int orc_attn_layer(void* h, int layer, const float* x, long B, long Tq, int causal_mask, int use_cache, float* y) {
    ORC_TRY
    auto* g = (OrcGpt*)h;
    Tensor in = Tensor::from(x, {B * Tq, (long)g->m.c.hidden});
    Tensor mask, maskE;
    if (causal_mask) {
        mask = Tensor(std::vector<long>{Tq, Tq}); buildtrimask(mask.p(), Tq, Tq, 0.0f, -30000.0f);
        maskE = mask.view({1, 1, Tq, Tq}).expand({B, (long)g->m.c.n_heads, Tq, Tq});
    }
    Tensor out = (g->m.c.attn_type == 1) ? gqa(g->m, layer, in, causal_mask ? &maskE : nullptr, B, use_cache ? &g->cache : nullptr)
                                         : mha(g->m, layer, in, causal_mask ? &maskE : nullptr, B, use_cache ? &g->cache : nullptr);
    std::memcpy(y, out.p(), sizeof(float) * out.count());
    ORC_CATCH
}
ORC_API int orc_ffn_layer(void* h, int layer, const float* x, long R, float* y) {
    ORC_TRY
    auto* g = (OrcGpt*)h;
    Tensor out = ffn(g->m, layer, Tensor::from(x, {R, (long)g->m.c.hidden}));
    std::memcpy(y, out.p(), sizeof(float) * out.count());
    ORC_CATCH
}
