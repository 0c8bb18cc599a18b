// Device kernels of the fused GPTDecoder path (gfx950).  Included by tship_gpt.hip only.
//
// Data layout in HBM
//   residual stream x      fp32 [rows][hidden]
//   GEMM inputs            model activation type AT (fp16 or fp32) [rows padded][K padded], zero padded
//   fp16 weights           "P32" packed: tile (nt, kt) = 32 output columns x 16 k, 1 KiB, stored as the
//                          A-operand fragment of v_mfma_f32_32x32x16_f16: lane l holds column nt*32 + l%32,
//                          k = kt*16 + 8*(l/32) .. +7.  All k-tiles of one column tile are contiguous, so a
//                          wavefront streams one contiguous range with 16-byte loads.
//   fp32 weights           row-major [K][N] as the reference stores them
//   KV cache               [layer][batch][kv_head][max_len][head_dim], keys after RoPE, head_dim contiguous
//   GEMM outputs           fp32 split-K partials [split][rows][N]; the consumer kernel adds them up in split
//                          order together with the bias, so results do not depend on scheduling.
#pragma once

#include "tship_internal.h"
#include <cstddef>
#include <type_traits>

namespace tship {

__device__ __forceinline__ float act_apply(int act, float w) {
    // TensorSharp/TensorApplyCPU.cs:1747-1801; act 3 is the reference's "SwiGLU" gate: no activation
    // (Seq2SeqSharp/Layers/PositionwiseFeedForward.cs:100-116)
    if (act == 0) return w < 0.0f ? 0.0f : w;
    if (act == 1 || act == 4) return w / (1.0f + __expf(-w));
    if (act == 2) return w < 0.0f ? 0.01f * w : w;
    return w;
}

// rotary embedding of one (even, odd) pair, two roundings per output like the reference's C# expression
// (TensorSharp/TensorApplyCPU.cs:1166-1173)
__device__ __forceinline__ void rope_pair(float x0, float x1, float c, float s, float& y0, float& y1) {
#pragma clang fp contract(off)
    y0 = x0 * c - x1 * s;
    y1 = x1 * c + x0 * s;
}

// op(v[l], v[l ^ 16]) and op(v[l], v[l ^ 32]) in every lane with v_permlane16_swap / v_permlane32_swap (gfx950): the swap
// of a register with its own copy leaves the lower partner's value in one result and the upper partner's in the other, in
// all lanes, so the reduction needs no trip through LDS (ds_bpermute: two dependent LDS round trips per softmax step) and
// adds the two partners in the same order in both lanes.
__device__ __forceinline__ float max_xor16(float v) {
    const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float max_xor32(float v) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float sum_xor16(float v) {
    const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float sum_xor32(float v) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// The same with the activation fixed at compile time: the epilogues of the LDS-tiled GEMM apply it to 64-128 values per lane,
// and a run-time switch per value is a chain of scalar compares and branches around each of them.
template <int ACT>
__device__ __forceinline__ float act_apply_c(float w) {
    if constexpr (ACT == 0) return w < 0.0f ? 0.0f : w;
    else if constexpr (ACT == 1 || ACT == 4) return w / (1.0f + __expf(-w));
    else if constexpr (ACT == 2) return w < 0.0f ? 0.01f * w : w;
    else return w;
}
// calls f(std::integral_constant<int, act>) for the run-time activation code
template <typename F>
__device__ __forceinline__ void with_act(int act, F&& f) {
    if (act == 0) f(std::integral_constant<int, 0>{});
    else if (act == 1 || act == 4) f(std::integral_constant<int, 1>{});
    else if (act == 2) f(std::integral_constant<int, 2>{});
    else f(std::integral_constant<int, 3>{});
}

// GEMM inputs of the fp16 decode path are stored "fragment packed": for every k-tile of 16 the 32 rows form the
// 1 KiB B-operand fragment of v_mfma_f32_32x32x16_f16 (lane l holds row l%32, k = kt*16 + 8*(l/32) .. +7), so a
// wavefront fetches it with one coalesced 16-byte load per lane.  Index of element (row b, column k):
__device__ __forceinline__ long xpack_index(int b, int k, int KT) {
    return ((((long)(b >> 5) * KT + (k >> 4)) * 64) + (b & 31) + 32 * ((k >> 3) & 1)) * 8 + (k & 7);
}

template <typename T> __device__ __forceinline__ float to_f32(T v) { return (float)v; }
template <typename T> __device__ __forceinline__ T from_f32(float v) { return (T)v; }

// ------------------------------------------------------------------------------------------------
// weight packing (runs once per tensor at load time)
// ------------------------------------------------------------------------------------------------
enum { PACK_PLAIN = 0, PACK_INTERLEAVE16 = 1 };

// src fp32 row-major [K][N] (ld) -> dst P32.  One thread per (source column, group of 8 k).
// PACK_PLAIN: destination column = n_off + n.  PACK_INTERLEAVE16: destination column =
// (n/16)*32 + n_off + n%16 with n_off in {0,16}: column tile j then holds 16 columns of the first matrix
// followed by the same 16 columns of the second, so a gated FFN epilogue finds both factors in one tile.
__global__ void pack_w_kernel(const float* __restrict__ src, long ld, int K, int N, half_t* __restrict__ dst, int KT,
                              int mode, int n_off) {
    long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    long total = (long)N * KT * 2;
    if (idx >= total) return;
    int n = (int)(idx % N);
    int kg = (int)(idx / N);
    int nd = mode == PACK_PLAIN ? n_off + n : (n / 16) * 32 + n_off + (n % 16);
    int nt = nd / 32, lane = (nd % 32) + 32 * (kg & 1), kt = kg >> 1;
    half8 v;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        int k = kg * 8 + j;
        v[j] = (half_t)(k < K ? src[(long)k * ld + n] : 0.0f);
    }
    *(half8*)(dst + (((long)nt * KT + kt) * 64 + lane) * 8) = v;
}

// fp32 -> T copy of a [rows][cols] matrix into a wider destination at a column offset
// Deferred LayerNorm: fold the norm's gamma and beta into per-column constants of a packed weight matrix (once, when the
// model is finalised).  For packed column n:  c[n] = sum_k gamma[k] W[k][n],  d[n] = sum_k beta[k] W[k][n] + bias(n),
// W being the fp16 values the GEMM multiplies with; sums in double, k ascending.  bias_mode 0: bias[n] (plain layout);
// 1: the gated interleave (packed column 32 g + j stands for column 16 g + j of W1 when j < 16, of W3 otherwise: bias1 /
// bias2); a null bias counts as zero.  One thread per packed column.
__global__ void ln_fold_kernel(const half_t* __restrict__ W, int KT, int NT, int K, const float* __restrict__ gamma, const float* __restrict__ beta,
                               const float* __restrict__ bias1, const float* __restrict__ bias2, int bias_mode, int n_logical,
                               float* __restrict__ c_out, float* __restrict__ d_out) {
    const int n = blockIdx.x * blockDim.x + threadIdx.x;
    if (n >= NT * 32) return;
    const int nt = n >> 5, nl = n & 31;
    double c = 0.0, d = 0.0;
    for (int k = 0; k < K; ++k) {
        const int kt = k >> 4, kl = k & 15, lane = nl + 32 * (kl >> 3), j = kl & 7;
        const double w = (double)(float)W[(((long)nt * KT + kt) * 64 + lane) * 8 + j];
        c += (double)gamma[k] * w;
        if (beta) d += (double)beta[k] * w;
    }
    float b = 0.0f;
    if (bias_mode == 0) { if (bias1 && n < n_logical) b = bias1[n]; }
    else {
        const int f = (n >> 5) * 16 + (n & 15);
        const float* src = (n & 16) ? bias2 : bias1;
        if (src && f < n_logical) b = src[f];
    }
    c_out[n] = (float)c;
    d_out[n] = (float)(d + (double)b);
}

template <typename T>
__global__ void copy_cols_kernel(const float* __restrict__ src, long ld_src, long rows, long cols, T* __restrict__ dst, long ld_dst,
                                 long col_off) {
    long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= rows * cols) return;
    long r = idx / cols, c = idx % cols;
    dst[r * ld_dst + col_off + c] = (T)src[r * ld_src + c];
}

// ------------------------------------------------------------------------------------------------
// decode GEMM, fp16 weights: Y[b][n] = sum_k X[b][k] * W[k][n] for <= 128 rows, MFMA 32x32x16.
// A block owns one 32-column tile and one k-split; its 4 wavefronts split the k range again and are
// reduced through LDS.  HBM-bound: every weight byte is read exactly once with 16-byte loads.
// ------------------------------------------------------------------------------------------------
enum { EPI_PARTIAL = 0, EPI_F32_BIAS = 1, EPI_ACT16 = 2, EPI_RESID_TAIL = 3, EPI_SPLIT_TAIL = 4 };

struct SkinnyArgs {
    const half_t* W; int KT; int NT;
    const half_t* X; int ldx;
    int KS;
    float* out; int ld_out; long split_stride;
    const float* bias; const float* bias2;
    half_t* out16; int ld16;
    int out16_kt;          // > 0: out16 is fragment packed with this many k-tiles per row block; 0: row-major with ld16
    int act; int gated; int n_valid; int rows_valid;
    // optional batch of independent problems (MoE experts) on blockIdx.y: weights from a pointer table,
    // activations / outputs at a fixed stride, row counts read on the device
    const half_t* const* Wtab; long x_estride; long out_estride; long out16_estride; const int* rows_tab;
    int row_tiles_z;       // batched problems only: blockIdx.z selects a 32-row tile (kernels instantiated for one row tile)
    // deferred RMSNorm: the input rows were stored as half(gamma * x); the epilogue multiplies row b by
    // 1 / sqrt(sum_t ssq[t][b] / h + eps), the factor the norm would have applied (exact up to rounding)
    const float* ssq; int ssq_nt; int ssq_ld; float inv_h; float eps;
    // deferred LayerNorm (ln != 0; LayerNormalization.Norm, kernel TensorSharp/TensorApplyCPU.cs:1360-1447): the producers
    // also store the tiles' plain sums, behind the sums of squares (ssq + ssq_nt * ssq_ld); a consumer rebuilds the
    // row's mean and 1 / sigma = 1 / sqrt(E[x^2] - mean^2 + eps) and computes
    //     Y = ((half(gamma x) W) - mean * c) / sigma + d,   c[n] = sum_k gamma[k] W[k][n],   d[n] = sum_k beta[k] W[k][n] + bias[n]
    // with c and d per packed output column (ln_c, ln_d; folded once, when the model is finalised), which is the
    // product of the normalised row with W.  The bias pointers are not read then.
    int ln; const float* ln_c; const float* ln_d;
    // EPI_RESID_TAIL (KS == 1: the block holds the complete sums of its column tile): adds bias and residual, stores
    // x, the next GEMM's packed input half(gamma * x) and the tile's per-row sum of squares
    float* x; int ldx_res; const float* gamma; half_t* xg16; int xg_kt; float* ssq_out; int ssq_out_ld;
    int* advance_pos;      // optional: one thread of the launch increments this device counter
    // EPI_SPLIT_TAIL (KS > 1): the KS blocks of a column tile exchange their partial sums through `out` with
    // agent-scope atomic stores and loads (they bypass the per-XCD L2, which is not coherent across XCDs for plain
    // accesses), count themselves in tile_count[nt], and the block that arrives last performs the epilogue
    int* tile_count;
};

// NW wavefronts per block work on the same 32-column tile and split the block's k range; every wavefront keeps
// 8 weight fragments and 8 activation fragments (16 KiB) in flight.  Accumulators are added pairwise through LDS
// (a fixed tree, so the sum order never changes); the last two are transposed through LDS so that the epilogue
// writes coalesced rows.  X is fragment packed (xpack_index).
// NJ > 1 (activation epilogue only): the block works on NJ neighbouring column tiles with one copy of the activation
// fragments.  A compute unit turns over a fixed number of requested bytes per microsecond, weights from HBM and
// activations from L2 alike, and a launch lasts as long as its busiest unit; 352 tiles of 32 columns on 256 units
// mean two tiles, twice 128 KiB of weights plus twice 128 KiB of activations, on the busiest ones.  176 blocks of two
// tiles request 256 + 128 KiB each.  HALF: a block takes one tile and half of a neighbour (three blocks' worth of
// tiles go to two blocks; 235 blocks of 192 + 128 KiB for 352 tiles).  A half tile is columns 0-7 and 16-23 of the
// tile, or 8-15 and 24-31: whole 128-byte runs of a weight fragment, and both factors of a gated pair (n, n + 16).
// The lanes of the other columns fetch their neighbours' bytes again (same cache lines, no further request) and
// compute sums that are never stored.
// The leading scalar arguments are the ones the first weight and activation requests depend on.  They are preloaded into
// scalar registers when the wavefront is created (the translation unit is compiled with a kernel-argument preload count;
// a struct passed by value is never preloaded), so those requests go out without a round trip to the argument segment;
// everything else arrives from the struct while they are in flight.  The struct's own copies of these fields are ignored.
// BATCHED: the launch covers several problems (MoE experts, a.Wtab / a.rows_tab); a template argument, because the branch
// would otherwise put a wait for the struct in front of every launch's first requests.
template <int BT, int EPI, int NW, int U = 8, int NJ = 1, bool HALF = false, bool BATCHED = false>
__global__ __launch_bounds__(NW * 64) void skinny_gemm_f16_kernel(const half_t* __restrict__ W_, const half_t* __restrict__ X_, int KT_, int NT_, int KS_,
                                                                  int rows_valid_, const float* __restrict__ ssq_, int ssq_nt_, int ssq_ld_, int ln_,
                                                                  SkinnyArgs a) {
    a.W = W_; a.X = X_; a.KT = KT_; a.NT = NT_; a.KS = KS_; a.rows_valid = rows_valid_; a.ssq = ssq_; a.ssq_nt = ssq_nt_; a.ssq_ld = ssq_ld_; a.ln = ln_;
    static_assert(!HALF || NJ == 2, "tile-and-a-half blocks are two-tile blocks with one tile half masked");
    static_assert(NJ == 1 || (EPI == EPI_ACT16 && BT == 1 && NW == 8), "several column tiles per block: one-round activation epilogue only");
    // one batch tile and eight wavefronts: every wavefront stores its accumulator once and the epilogue adds the eight
    // copies in wavefront order (one barrier); otherwise a pairwise tree followed by a transpose
    constexpr bool ONE_ROUND = BT == 1 && NW == 8 && (EPI == EPI_ACT16 || EPI == EPI_RESID_TAIL || EPI == EPI_SPLIT_TAIL);   // fp32 outputs keep the transpose: coalesced rows
    constexpr int RED = (ONE_ROUND ? NW : NW / 2) * BT * 16 * 64, FIN = 2 * BT * 32 * 33;
    __shared__ float smem[RED > FIN ? RED : FIN];      // the tree buffers are dead when the transpose buffer is written
    float (*red)[BT][16][64] = (float (*)[BT][16][64])smem;
    float (*fin)[BT * 32][33] = (float (*)[BT * 32][33])smem;
    unsigned bx = blockIdx.x;           // the block's place along x (column tiles x splits), remapped for batched launches
    if constexpr (BATCHED) {
        int e = blockIdx.y, rtz = blockIdx.z;
        if ((gridDim.y & 7) == 0 && !a.row_tiles_z) {
            // Blocks go to the XCDs round robin in dispatch order (x fastest).  With the column tiles of one problem spread
            // over all eight XCDs every XCD's L2 fetches every problem's activation tiles (measured: 15 % more bytes than
            // the weights at 8 experts x 64 rows).  Here XCD i takes problems i, i + 8, ... whole: the j-th block that lands
            // on an XCD is column tile j % gridDim.x of its (j / gridDim.x)-th problem.  Not for launches with a block per
            // row tile (row_tiles_z): a problem with more than 32 rows has more blocks that do work there, and the XCD that
            // held it alone made the launch 37 % longer; with only the first plane remapped the launch measured the same
            // as without.
            const unsigned id = blockIdx.x + gridDim.x * blockIdx.y;
            const unsigned xcd = id & 7, j = id >> 3, per = gridDim.y >> 3;
            bx = j % gridDim.x;
            e = (int)(xcd + 8 * ((j / gridDim.x) % per));
        }
        a.rows_valid = a.rows_tab[e];
        if (a.row_tiles_z) {
            // one 32-row tile per block, tile number on blockIdx.z: an expert with at most 32 rows (the usual case at decode)
            // costs one block per column tile, the blocks of its empty row tiles leave at once; an expert with more rows
            // has its weights streamed once per row tile
            const int rt = rtz;
            a.rows_valid -= 32 * rt;
            a.X += (long)rt * a.KT * 512;
            if (a.out) a.out += (long)rt * 32 * a.ld_out;
            if (a.out16) a.out16 += a.out16_kt > 0 ? (long)rt * a.out16_kt * 512 : (long)rt * 32 * a.ld16;
        }
        if (a.rows_valid <= 0) return;
        a.W = a.Wtab[e]; a.X += e * a.x_estride;
        if (a.out) a.out += e * a.out_estride;
        if (a.out16) a.out16 += e * a.out16_estride;
    }
    const int lane = threadIdx.x & 63, w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int ks = bx % a.KS;
    // tile of slot j, and for a half tile which one: 0 whole, 1 columns 0-7 / 16-23, 2 columns 8-15 / 24-31
    int tile_of[NJ], half_of[NJ];
    if constexpr (HALF) {
        const int grp = bx >> 1, odd = bx & 1, whole = (a.NT / 3) * 2;
        if ((int)bx < whole) {
            tile_of[0] = 3 * grp + odd; half_of[0] = odd ? 2 : 0;
            tile_of[1] = 3 * grp + 1 + odd; half_of[1] = odd ? 0 : 1;
        } else {      // the one or two tiles left over: a block each
            tile_of[0] = 3 * (a.NT / 3) + ((int)bx - whole); half_of[0] = 0;
            tile_of[1] = a.NT; half_of[1] = 0;
        }
    } else {
#pragma unroll
        for (int j = 0; j < NJ; ++j) { tile_of[j] = (bx / a.KS) * NJ + j; half_of[j] = 0; }
    }
    const int nt = tile_of[0];
    const int per = (a.KT + a.KS - 1) / a.KS;
    const int k0 = ks * per, k1 = min(a.KT, k0 + per);
    const int pw = (max(k1 - k0, 0) + NW - 1) / NW;
    const int wk0 = k0 + w * pw, wk1 = min(k1, wk0 + pw);

    floatx16 acc[NJ][BT];
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
        for (int bt = 0; bt < BT; ++bt)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[j][bt][v] = 0.0f;

    // deferred-norm inputs: this thread's share of the per-tile sums of squares, fetched before the weight stream
    __shared__ float srinv[BT * 32];
    constexpr int NCH = (NW * 64) / (BT * 32);
    __shared__ float schunk[NCH][BT * 32];
    __shared__ float schunk2[NCH][BT * 32];      // LayerNorm: the plain sums' chunks
    __shared__ float smean[BT * 32];
    // (the first eight tile sums of a chunk are requested here and stay in registers until the weight stream has been
    // requested, so that their latency hides behind it; a chunk's tail beyond eight tiles is added behind the stream)
    float ssq_v[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    float ssum_v[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};      // (LayerNorm: the tiles' plain sums)
    if (a.ssq) {
        const int b = threadIdx.x % (BT * 32), ch = threadIdx.x / (BT * 32);
        const int per_ch = (a.ssq_nt + NCH - 1) / NCH;
        const int t0 = ch * per_ch, t1 = min(a.ssq_nt, t0 + per_ch);
        // (unconditional requests at clamped tiles; what lies beyond the chunk is dropped)
        // (the values stay untouched until they are added behind the stream: any arithmetic on them here would wait for them)
        (void)t1;
        const long sum_off = (long)a.ssq_nt * a.ssq_ld;
        if (per_ch > 4) {
#pragma unroll
            for (int i = 0; i < 8; ++i) ssq_v[i] = a.ssq[(long)min(t0 + i, a.ssq_nt - 1) * a.ssq_ld + b];
            if (a.ln) {
#pragma unroll
                for (int i = 0; i < 8; ++i) ssum_v[i] = a.ssq[sum_off + (long)min(t0 + i, a.ssq_nt - 1) * a.ssq_ld + b];
            }
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) ssq_v[i] = a.ssq[(long)min(t0 + i, a.ssq_nt - 1) * a.ssq_ld + b];
            if (a.ln) {
#pragma unroll
                for (int i = 0; i < 4; ++i) ssum_v[i] = a.ssq[sum_off + (long)min(t0 + i, a.ssq_nt - 1) * a.ssq_ld + b];
            }
        }
    }
    // (a tile beyond the last one reads the last one again; nothing of it is stored)
    const half_t* wp[NJ];
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        // lane l feeds column l % 32 of the tile; the lanes outside a half tile read what their neighbours 8 columns away read
        const int src = half_of[j] == 1 ? (lane & ~8) : half_of[j] == 2 ? (lane | 8) : lane;
        wp[j] = a.W + ((long)min(tile_of[j], a.NT - 1) * a.KT * 64 + src) * 8;
    }
    // Activation fragments: lane l holds row l % 32 of a 32-row tile.  Rows from rows_valid on need no bytes of their
    // own: their lanes read the bytes of valid rows again (whole 8-lane, 128-byte runs; row tiles without a valid row
    // read the last tile that has one), which costs no further request, and their sums are never stored.
    const half_t* xp[BT];
    {
        const int rv = max(a.rows_valid, 1), last_bt = min((rv - 1) >> 5, BT - 1);
        const int rv8 = min(32, (rv - last_bt * 32 + 7) & ~7);
        const int dup = (lane & 32) | ((lane & 31) % rv8);
#pragma unroll
        for (int bt = 0; bt < BT; ++bt) xp[bt] = a.X + (long)min(bt, last_bt) * a.KT * 512 + (bt >= last_bt ? dup : lane) * 8;
    }
    // Full batches of U k-tiles run without conditions: a request under a condition of its own would make every
    // later wait cover all requests, and the products could not start while the batch is still arriving.
    int kt = wk0;
    // The first batch is requested before anything that needs the argument struct: its addresses come from preloaded
    // arguments only.  Its requests are unconditional (k-tiles beyond the wavefront's range are clamped into the matrix and
    // their fragments dropped), so that the waits stay exact.
    half8 wf0[U][NJ];
    half8 xf0[U][BT];
    {
        const int klast = max(min(wk1, a.KT) - 1, 0);
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int kk = min(kt + u, klast);
#pragma unroll
            for (int j = 0; j < NJ; ++j) wf0[u][j] = load_once((const half8*)(wp[j] + (long)kk * 512));
#pragma unroll
            for (int bt = 0; bt < BT; ++bt) xf0[u][bt] = *(const half8*)(xp[bt] + (long)kk * 512);
        }
    }
    __builtin_amdgcn_sched_barrier(0);
    // bias of this thread's outputs in the one-round activation epilogue
    float eb1[NJ], eb2[NJ], ec1[NJ], ec2[NJ];      // (ec: LayerNorm's column sums c of the thread's outputs, 0 otherwise)
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        eb1[j] = 0.0f; eb2[j] = 0.0f; ec1[j] = 0.0f; ec2[j] = 0.0f;
        if (ONE_ROUND && EPI == EPI_ACT16) {
            const int n1 = 8 * (w >> 2) + 4 * (lane >> 5) + (w & 3);
            // (unconditional requests at clamped indices: a request under a condition of its own, issued between the first
            // batch's requests and its products, would make the waits for the batch inexact)
            const int nlast = max(a.n_valid, 1) - 1;
            if (a.ln) {
                // per packed column (the tile's columns n1 and n1 + 16, whatever they stand for)
                const int pc = min(tile_of[j], a.NT - 1) * 32 + n1;
                eb1[j] = a.ln_d[pc]; eb2[j] = a.ln_d[pc + 16]; ec1[j] = a.ln_c[pc]; ec2[j] = a.ln_c[pc + 16];
            } else if (a.gated) {
                const int f = tile_of[j] * 16 + n1;
                eb1[j] = a.bias[min(f, nlast)]; eb2[j] = a.bias2[min(f, nlast)];      // (used only where f < n_valid)
            } else {
                const int f = tile_of[j] * 32 + n1;
                eb1[j] = a.bias[min(f, nlast)]; eb2[j] = a.bias[min(f + 16, nlast)];  // (used only where the column is valid)
            }
        }
    }
    // residual tail: the old residual, bias and gamma of this thread's outputs do not depend on the product
    constexpr int ITER = BT * 1024 / (NW * 64);
    float tail_x[ITER], tail_b[ITER], tail_g[ITER];
    if (EPI == EPI_RESID_TAIL || EPI == EPI_SPLIT_TAIL) {
#pragma unroll
        for (int it = 0; it < ITER; ++it) {
            const int idx = threadIdx.x + it * NW * 64;
            // (one-round epilogue: outputs (lane % 32, n1) and (lane % 32, n1 + 16); otherwise row-major over the tile)
            const int col = nt * 32 + (ONE_ROUND ? 8 * (w >> 2) + 4 * (lane >> 5) + (w & 3) + 16 * it : (idx & 31));
            const int b = ONE_ROUND ? (lane & 31) : (idx >> 5);
            // (unconditional requests at clamped indices, see above; the values are used only for valid rows and columns)
            const int bc = min(b, max(a.rows_valid, 1) - 1), cc = min(col, max(a.n_valid, 1) - 1);
            tail_x[it] = a.x[(long)bc * a.ldx_res + cc];
            tail_b[it] = a.bias[cc];
            tail_g[it] = a.gamma[cc];
        }
    }
    __builtin_amdgcn_sched_barrier(0);
    if (kt + U <= wk1) {
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int j = 0; j < NJ; ++j)
#pragma unroll
                for (int bt = 0; bt < BT; ++bt) acc[j][bt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf0[u][j], xf0[u][bt], acc[j][bt], 0, 0, 0);
    } else {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (kt + u < wk1) {
#pragma unroll
                for (int j = 0; j < NJ; ++j)
#pragma unroll
                    for (int bt = 0; bt < BT; ++bt) acc[j][bt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf0[u][j], xf0[u][bt], acc[j][bt], 0, 0, 0);
            }
        }
    }
    kt = min(kt + U, max(wk1, wk0));
    __builtin_amdgcn_sched_barrier(0);
    for (; kt + U <= wk1; kt += U) {
        half8 wf[U][NJ];
        half8 xf[U][BT];
#pragma unroll
        for (int u = 0; u < U; ++u) {
#pragma unroll
            for (int j = 0; j < NJ; ++j) wf[u][j] = load_once((const half8*)(wp[j] + (long)(kt + u) * 512));
#pragma unroll
            for (int bt = 0; bt < BT; ++bt) xf[u][bt] = *(const half8*)(xp[bt] + (long)(kt + u) * 512);
        }
        __builtin_amdgcn_sched_barrier(0);       // all requests of the batch go out before its first product
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int j = 0; j < NJ; ++j)
#pragma unroll
                for (int bt = 0; bt < BT; ++bt) acc[j][bt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf[u][j], xf[u][bt], acc[j][bt], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
    }
    if (kt < wk1) {
        half8 wf[U][NJ];
        half8 xf[U][BT];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (kt + u < wk1) {
#pragma unroll
                for (int j = 0; j < NJ; ++j) wf[u][j] = load_once((const half8*)(wp[j] + (long)(kt + u) * 512));
#pragma unroll
                for (int bt = 0; bt < BT; ++bt) xf[u][bt] = *(const half8*)(xp[bt] + (long)(kt + u) * 512);
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (kt + u < wk1) {
#pragma unroll
                for (int j = 0; j < NJ; ++j)
#pragma unroll
                    for (int bt = 0; bt < BT; ++bt) acc[j][bt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf[u][j], xf[u][bt], acc[j][bt], 0, 0, 0);
            }
        }
    }
    // rinv per row from the tile sums: NCH chunks of tiles are added in parallel (loads issued before the weight
    // stream, see above), then the chunk sums in order
    if (a.ssq) {
        float ssq_part = 0.0f;
        {
            const int b = threadIdx.x % (BT * 32), ch = threadIdx.x / (BT * 32);
            const int per_ch = (a.ssq_nt + NCH - 1) / NCH;
            const int t0 = ch * per_ch, t1 = min(a.ssq_nt, t0 + per_ch);
#pragma unroll
            for (int i = 0; i < 8; ++i) ssq_part += (i < (per_ch > 4 ? 8 : 4) && t0 + i < t1) ? ssq_v[i] : 0.0f;
            for (int t = t0 + 8; t < t1; t += 8) {       // (wide models at batches above 32: eight independent requests at a time)
                float v[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) v[i] = a.ssq[(long)min(t + i, a.ssq_nt - 1) * a.ssq_ld + b];
#pragma unroll
                for (int i = 0; i < 8; ++i) ssq_part += t + i < t1 ? v[i] : 0.0f;
            }
        }
        schunk[threadIdx.x / (BT * 32)][threadIdx.x % (BT * 32)] = ssq_part;
        if (a.ln) {
            float ssum_part = 0.0f;
            const int b = threadIdx.x % (BT * 32), ch = threadIdx.x / (BT * 32);
            const int per_ch = (a.ssq_nt + NCH - 1) / NCH;
            const int t0 = ch * per_ch, t1 = min(a.ssq_nt, t0 + per_ch);
            const long sum_off = (long)a.ssq_nt * a.ssq_ld;
#pragma unroll
            for (int i = 0; i < 8; ++i) ssum_part += (i < (per_ch > 4 ? 8 : 4) && t0 + i < t1) ? ssum_v[i] : 0.0f;
            for (int t = t0 + 8; t < t1; ++t) ssum_part += a.ssq[sum_off + (long)t * a.ssq_ld + b];
            schunk2[threadIdx.x / (BT * 32)][threadIdx.x % (BT * 32)] = ssum_part;
        }
        __syncthreads();
        if (threadIdx.x < BT * 32) {
            float tot = 0.0f;
#pragma unroll
            for (int c = 0; c < NCH; ++c) tot += schunk[c][threadIdx.x];
            if (a.ln) {
                float tots = 0.0f;
#pragma unroll
                for (int c = 0; c < NCH; ++c) tots += schunk2[c][threadIdx.x];
                const float mean = tots * a.inv_h;
                srinv[threadIdx.x] = 1.0f / sqrtf(fmaxf(tot * a.inv_h - mean * mean, 0.0f) + a.eps);
                smean[threadIdx.x] = mean;
            } else {
                srinv[threadIdx.x] = 1.0f / sqrtf(tot * a.inv_h + a.eps);
                smean[threadIdx.x] = 0.0f;
            }
        }
    }
    if (a.advance_pos && blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) { a.advance_pos[0] += 1; a.advance_pos[1] += 1; }
    if constexpr (ONE_ROUND && NJ > 1) {
        // the column tiles one after the other through the same LDS buffer
        const int b = lane & 31, n1 = 8 * (w >> 2) + 4 * (lane >> 5) + (w & 3);
        const bool rok = b < a.rows_valid;
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            if (tile_of[j] >= a.NT) break;
            if (j) __syncthreads();
#pragma unroll
            for (int v = 0; v < 16; ++v) red[w][0][v][lane] = acc[j][0][v];
            __syncthreads();
            float s1 = red[0][0][w][lane], s2 = red[0][0][w + 8][lane];
#pragma unroll
            for (int i = 1; i < NW; ++i) { s1 += red[i][0][w][lane]; s2 += red[i][0][w + 8][lane]; }
            const float rinv = a.ssq ? srinv[b] : 1.0f, mean = a.ssq ? smean[b] : 0.0f;
            s1 -= mean * ec1[j]; s2 -= mean * ec2[j];       // (LayerNorm: the mean's share of the product; 0 otherwise)
            // (outputs n1 and n1 + 16 belong to the first half of a tile when n1 < 8)
            const bool mine = half_of[j] == 0 || (half_of[j] == 1) == (n1 < 8);
            if (a.gated) {
                const int f = tile_of[j] * 16 + n1;
                if (rok && mine && f < a.n_valid) {
                    const float val = act_apply(a.act, s1 * rinv + eb1[j]) * (s2 * rinv + eb2[j]);
                    if (a.out16_kt > 0) a.out16[xpack_index(b, f, a.out16_kt)] = (half_t)val;
                    else a.out16[(long)b * a.ld16 + f] = (half_t)val;
                }
            } else {
#pragma unroll
                for (int q = 0; q < 2; ++q) {
                    const int f = tile_of[j] * 32 + n1 + 16 * q;
                    if (rok && mine && f < a.n_valid) {
                        const float val = act_apply(a.act, (q ? s2 : s1) * rinv + (q ? eb2[j] : eb1[j]));
                        if (a.out16_kt > 0) a.out16[xpack_index(b, f, a.out16_kt)] = (half_t)val;
                        else a.out16[(long)b * a.ld16 + f] = (half_t)val;
                    }
                }
            }
        }
        return;
    } else if constexpr (ONE_ROUND) {
#pragma unroll
        for (int v = 0; v < 16; ++v) red[w][0][v][lane] = acc[0][0][v];
        __syncthreads();
        // thread (wavefront w, lane): registers v = w and w + 8 of all eight copies -> batch row lane % 32, columns
        // n1 = 8 (w / 4) + 4 (lane / 32) + w % 4 and n1 + 16 (the gate's two factors when the tile is interleaved)
        float s1 = red[0][0][w][lane], s2 = red[0][0][w + 8][lane];
#pragma unroll
        for (int i = 1; i < NW; ++i) { s1 += red[i][0][w][lane]; s2 += red[i][0][w + 8][lane]; }
        const int b = lane & 31, n1 = 8 * (w >> 2) + 4 * (lane >> 5) + (w & 3);
        const bool rok = b < a.rows_valid;
        const float rinv = a.ssq ? srinv[b] : 1.0f, mean = a.ssq ? smean[b] : 0.0f;
        if (EPI == EPI_ACT16) { s1 -= mean * ec1[0]; s2 -= mean * ec2[0]; }      // (LayerNorm: the mean's share of the product; 0 otherwise)
        if (EPI == EPI_SPLIT_TAIL) {
            // publish this block's partial sums, then find out whether it is the last of its column tile
            //
            // Memory model: the C++ model would want a release on the counter add and an acquire in the last block; that
            // fence costs a write-back of the whole L2 here (measured > 10 us).  What this code relies on instead is the
            // instruction sequence itself, on gfx950 (the build refuses other targets, tship_internal.h):
            //   1. the data stores are agent-scope atomic stores: global_store_dword ... sc1, written through to the point of
            //      coherence shared by the XCDs' L2s;
            //   2. s_waitcnt vmcnt(0) (the asm below; "memory" keeps the compiler from moving accesses across it): vmcnt
            //      counts stores on this target, so every store of this wavefront has been acknowledged there;
            //   3. the block barrier: all wavefronts of the block are past (2);
            //   4. one thread's agent-scope atomic add on the tile's counter: performed at that same point of coherence,
            //      after this block's data;
            //   5. the last arriver (control dependent on the counter's value, which no wavefront has before its
            //      s_waitcnt for the returned data) reads all partials with agent-scope atomic loads (... sc1: they do
            //      not hit stale lines of its own L2).
            // The counter is back at zero when the launch ends, and is cleared by TSHip_GptReset and before graph capture.
            __shared__ int s_last;
            // (exchange layout [split][tile][2][512 threads]: a wavefront's store is 256 contiguous bytes)
            float* o = a.out + ((long)ks * a.NT + nt) * 1024 + threadIdx.x;
            __hip_atomic_store(o, s1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(o + 512, s2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");            // the stores have reached the point of coherence
            __syncthreads();
            if (threadIdx.x == 0) s_last = __hip_atomic_fetch_add(a.tile_count + nt, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == a.KS - 1;
            __syncthreads();
            if (!s_last) return;
            // every block of the tile has published (its count came after its stores): add the KS partials in order
            const float* p = a.out + (long)nt * 1024 + threadIdx.x;
            const long sstride = (long)a.NT * 1024;
            float p1[8], p2[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                p1[k] = k < a.KS ? __hip_atomic_load(p + k * sstride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0.0f;
                p2[k] = k < a.KS ? __hip_atomic_load(p + k * sstride + 512, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0.0f;
            }
            s1 = p1[0]; s2 = p2[0];
#pragma unroll
            for (int k = 1; k < 8; ++k) if (k < a.KS) { s1 += p1[k]; s2 += p2[k]; }
            for (int k = 8; k < a.KS; ++k) {
                s1 += __hip_atomic_load(p + k * sstride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                s2 += __hip_atomic_load(p + k * sstride + 512, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            if (threadIdx.x == 0) __hip_atomic_store(a.tile_count + nt, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // ready for the next launch
        }
        if (EPI == EPI_PARTIAL) {
            if (rok) {
                float* o = a.out + ks * a.split_stride + (long)b * a.ld_out + nt * 32 + n1;
                o[0] = s1; o[16] = s2;
            }
        } else if (EPI == EPI_F32_BIAS) {
            const int c1 = nt * 32 + n1, c2 = c1 + 16;
            if (a.ln) {
                if (rok && c1 < a.n_valid) a.out[(long)b * a.ld_out + c1] = (s1 - mean * a.ln_c[c1]) * rinv + a.ln_d[c1];
                if (rok && c2 < a.n_valid) a.out[(long)b * a.ld_out + c2] = (s2 - mean * a.ln_c[c2]) * rinv + a.ln_d[c2];
            } else {
            if (rok && c1 < a.n_valid) a.out[(long)b * a.ld_out + c1] = s1 * rinv + a.bias[c1];
            if (rok && c2 < a.n_valid) a.out[(long)b * a.ld_out + c2] = s2 * rinv + a.bias[c2];
            }
        } else if (EPI == EPI_ACT16) {
            if (a.gated) {
                const int f = nt * 16 + n1;
                if (rok && f < a.n_valid) {
                    const float val = act_apply(a.act, s1 * rinv + eb1[0]) * (s2 * rinv + eb2[0]);
                    if (a.out16_kt > 0) a.out16[xpack_index(b, f, a.out16_kt)] = (half_t)val;
                    else a.out16[(long)b * a.ld16 + f] = (half_t)val;
                }
            } else {
#pragma unroll
                for (int q = 0; q < 2; ++q) {
                    const int f = nt * 32 + n1 + 16 * q;
                    if (rok && f < a.n_valid) {
                        const float val = act_apply(a.act, (q ? s2 : s1) * rinv + (q ? eb2[0] : eb1[0]));
                        if (a.out16_kt > 0) a.out16[xpack_index(b, f, a.out16_kt)] = (half_t)val;
                        else a.out16[(long)b * a.ld16 + f] = (half_t)val;
                    }
                }
            }
        } else {      // EPI_RESID_TAIL, EPI_SPLIT_TAIL
            __shared__ float sq[NW][32];
            __shared__ float ssm[NW][32];
            float q = 0.0f, sv = 0.0f;
#pragma unroll
            for (int h2 = 0; h2 < 2; ++h2) {
                const int col = nt * 32 + n1 + 16 * h2;
                if (rok && col < a.n_valid) {
                    const float v = ((h2 ? s2 : s1) + tail_b[h2]) + tail_x[h2];
                    a.x[(long)b * a.ldx_res + col] = v;
                    a.xg16[xpack_index(b, col, a.xg_kt)] = (half_t)(tail_g[h2] * v);
                    q += v * v; sv += v;
                }
            }
            q += __shfl_xor(q, 32, 64);           // the two lane halves hold different columns of the same row
            if (lane < 32) sq[w][lane] = q;
            if (a.ln) { sv += __shfl_xor(sv, 32, 64); if (lane < 32) ssm[w][lane] = sv; }
            __syncthreads();
            if (threadIdx.x < 32 && threadIdx.x < a.rows_valid) {
                float tot = sq[0][threadIdx.x];
#pragma unroll
                for (int i = 1; i < NW; ++i) tot += sq[i][threadIdx.x];
                a.ssq_out[(long)nt * a.ssq_out_ld + threadIdx.x] = tot;
                if (a.ln) {      // the tile's plain sum, behind the NT tiles of sums of squares
                    float tots = ssm[0][threadIdx.x];
#pragma unroll
                    for (int i = 1; i < NW; ++i) tots += ssm[i][threadIdx.x];
                    a.ssq_out[((long)a.NT + nt) * a.ssq_out_ld + threadIdx.x] = tots;
                }
            }
        }
        return;
    }
    // pairwise tree over wavefronts down to two: in each round the upper half stores, the lower half adds
#pragma unroll
    for (int half = NW / 2; half >= 2; half >>= 1) {
        if (w >= half && w < 2 * half) {
#pragma unroll
            for (int bt = 0; bt < BT; ++bt)
#pragma unroll
                for (int v = 0; v < 16; ++v) red[w - half][bt][v][lane] = acc[0][bt][v];
        }
        __syncthreads();
        if (w < half) {
#pragma unroll
            for (int bt = 0; bt < BT; ++bt)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[0][bt][v] += red[w][bt][v][lane];
        }
        __syncthreads();
    }
    // accumulator lane l, register v: column nt*32 + 8*(v/4) + 4*(l/32) + v%4 of batch row bt*32 + l%32
    if (w < 2) {
#pragma unroll
        for (int bt = 0; bt < BT; ++bt)
#pragma unroll
            for (int v = 0; v < 16; ++v) fin[w][bt * 32 + (lane & 31)][8 * (v / 4) + 4 * (lane >> 5) + (v % 4)] = acc[0][bt][v];
    }
    __syncthreads();
    float keep[ITER];
#pragma unroll
    for (int it = 0; it < ITER; ++it) {
        const int idx = threadIdx.x + it * NW * 64;
        const int n = idx & 31, b = idx >> 5;
        keep[it] = 0.0f;
        if (b >= a.rows_valid) continue;
        float s = fin[0][b][n] + fin[1][b][n];
        const float rinv = a.ssq ? srinv[b] : 1.0f;
        if (EPI == EPI_PARTIAL) {
            a.out[ks * a.split_stride + (long)b * a.ld_out + nt * 32 + n] = s;
        } else if (EPI == EPI_RESID_TAIL) {
            keep[it] = s;
        } else if (EPI == EPI_F32_BIAS) {
            const int col = nt * 32 + n;
            if (col < a.n_valid) a.out[(long)b * a.ld_out + col] = a.ln ? (s - smean[b] * a.ln_c[col]) * rinv + a.ln_d[col] : s * rinv + a.bias[col];
        } else {
            float val; int f; bool ok;
            if (a.gated) {
                const float c = fin[0][b][(n & 15) + 16] + fin[1][b][(n & 15) + 16];
                f = nt * 16 + n; ok = n < 16 && f < a.n_valid;
                val = ok ? act_apply(a.act, s * rinv + a.bias[f]) * (c * rinv + a.bias2[f]) : 0.0f;
            } else {
                f = nt * 32 + n; ok = f < a.n_valid;
                val = ok ? act_apply(a.act, s * rinv + a.bias[f]) : 0.0f;
            }
            if (ok) {
                if (a.out16_kt > 0) a.out16[xpack_index(b, f, a.out16_kt)] = (half_t)val;
                else a.out16[(long)b * a.ld16 + f] = (half_t)val;
            }
        }
    }
    if (EPI != EPI_RESID_TAIL) return;
#pragma unroll
    for (int it = 0; it < ITER; ++it) {
        const int idx = threadIdx.x + it * NW * 64;
        const int n = idx & 31, b = idx >> 5;
        if (b >= a.rows_valid) continue;                      // uniform over the 32 lanes that share a row
        const int col = nt * 32 + n;
        float v = keep[it];
        float q = 0.0f;
        if (col < a.n_valid) {
            v = (v + tail_b[it]) + tail_x[it];
            a.x[(long)b * a.ldx_res + col] = v;
            a.xg16[xpack_index(b, col, a.xg_kt)] = (half_t)(tail_g[it] * v);
            q = v * v;
        }
#pragma unroll
        for (int o = 16; o > 0; o >>= 1) q += __shfl_xor(q, o, 64);
        if (n == 0) a.ssq_out[(long)nt * a.ssq_out_ld + b] = q;
    }
}

// ------------------------------------------------------------------------------------------------
// prefill GEMM, fp16 weights: many rows.  Block tile 128 rows x 128 columns; each wavefront owns one
// 32-column weight tile (streamed from HBM/L2 as packed fragments) and 4 row tiles.  MFMA-bound.
// ------------------------------------------------------------------------------------------------
enum { BEPI_F32_BIAS = 0, BEPI_RESID = 1, BEPI_ACT16 = 2 };

struct BigArgs {
    const half_t* W; int KT; int NT;
    const half_t* X; int ldx; int R;
    float* out; int ld_out;
    const float* bias; const float* bias2;
    half_t* out16; int ld16;
    int act; int gated; int n_valid;
    // deferred RMSNorm (LDS-tiled kernels only).  Consumers: X holds half(gamma * x) and every output row is scaled by
    // rinv[row] before the bias.  Producers (BEPI_RESID): besides the residual stream, store half(gamma * x) row-major
    // into xg16 and the sum of squares of every (32-column tile, row) into ssq_out[tile * ssq_ld + row].
    const float* rinv;
    half_t* xg16; int ld_xg; const float* gamma; float* ssq_out; long ssq_ld;
    // QKV projection of a prefill (BEPI_F32_BIAS, LDS-tiled kernel) writing the cache itself: columns from kv_col0 on are
    // kv_gd key columns, then kv_gd value columns (head size kv_D, both counts multiples of 128); row r is position
    // kv_pos0 + r % kv_Tq of sequence r / kv_Tq (kv_pos0 and kv_Tq multiples of 32).  Keys are rotated (rope_cos /
    // rope_sin [position][kv_D / 2], null: not) and both leave as whole fragments of the fragment-major fp16 cache
    // [sequence][kv_hkv heads][kv_max_len x kv_D]; only the query columns are stored to `out`.  kcache null: off.
    half_t* kcache; half_t* vcache; long kv_max_len; int kv_col0, kv_gd, kv_D, kv_hkv, kv_Tq, kv_pos0;
    const float* rope_cos; const float* rope_sin;
    // Several independent problems in one launch of the LDS-tiled kernel (the experts of a MoE layer at prefill): problem
    // e = blockIdx.x / blocks_per_problem takes its weights from Wtab[e], its row count from rows_tab[e] (read on the
    // device; blocks beyond it leave at once) and its activations / outputs at fixed strides.  0: one problem.
    int blocks_per_problem; const half_t* const* Wtab; const int* rows_tab; long x_estride, out_estride, out16_estride;
    // The same with the problems' row tiles packed one behind the other (packed_problems > 0; blocks_per_problem unused): the
    // launch covers packed_rt row tiles, an upper bound of the sum over the problems of ceil(rows_tab[e] / 256) that the host
    // knows without reading the counts (the sum of the rows / 256 + the number of problems); every block finds its problem
    // from the counts, blocks beyond the last problem's tiles leave at once.  Consecutive row tiles mostly belong to one
    // problem, so a patch still shares its weight tiles.
    int packed_problems; int packed_rt;
    // Optional (LDS-tiled asynchronous kernel): row r of problem e is row row_idx[e * idx_estride + r] of X (the rows an
    // expert was given, read where they lie instead of being copied together first)
    const int* row_idx; long idx_estride;
    // LDS-tiled asynchronous kernel: row tiles per XCD patch (8, or fewer for launches that would otherwise fill fewer
    // than eight patches and leave XCDs idle); 0 means 8
    int patch_rows;
};

template <int EPI>
__global__ __launch_bounds__(256) void big_gemm_f16_kernel(BigArgs a) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int nt = blockIdx.x * 4 + w;
    if (nt >= a.NT) return;
    const int row0 = blockIdx.y * 128;
    floatx16 acc[4];
#pragma unroll
    for (int rt = 0; rt < 4; ++rt)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[rt][v] = 0.0f;
    const half_t* wp = a.W + ((long)nt * a.KT * 64 + lane) * 8;
    const half_t* xp = a.X + (long)(row0 + (lane & 31)) * a.ldx + (lane >> 5) * 8;
#pragma unroll 2
    for (int kt = 0; kt < a.KT; ++kt) {
        half8 wf = *(const half8*)(wp + (long)kt * 512);
        half8 xf[4];
#pragma unroll
        for (int rt = 0; rt < 4; ++rt) xf[rt] = *(const half8*)(xp + (long)rt * 32 * a.ldx + kt * 16);
#pragma unroll
        for (int rt = 0; rt < 4; ++rt) acc[rt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf, xf[rt], acc[rt], 0, 0, 0);
    }
#pragma unroll
    for (int rt = 0; rt < 4; ++rt) {
        const int row = row0 + rt * 32 + (lane & 31);
        if (row >= a.R) continue;
        if (EPI == BEPI_ACT16 && a.gated) {
#pragma unroll
            for (int v = 0; v < 8; ++v) {
                int nl = 8 * (v / 4) + 4 * (lane >> 5) + (v % 4);
                int f = nt * 16 + nl;
                if (f < a.n_valid)
                    a.out16[(long)row * a.ld16 + f] = (half_t)(act_apply(a.act, acc[rt][v] + a.bias[f]) * (acc[rt][v + 8] + a.bias2[f]));
            }
        } else {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                int col = nt * 32 + 8 * (v / 4) + 4 * (lane >> 5) + (v % 4);
                if (col >= a.n_valid) continue;
                float s = acc[rt][v] + a.bias[col];
                if (EPI == BEPI_F32_BIAS) a.out[(long)row * a.ld_out + col] = s;
                else if (EPI == BEPI_RESID) a.out[(long)row * a.ld_out + col] = s + a.out[(long)row * a.ld_out + col];
                else a.out16[(long)row * a.ld16 + col] = (half_t)act_apply(a.act, s);
            }
        }
    }
}

// Epilogue shared by the LDS-tiled prefill GEMMs.
// Gated activation output of one wavefront (64 rows x 4 column tiles = 64 consecutive fp16 outputs per row) through LDS, so
// that rows leave as whole 128-byte lines (eight lanes x 16 bytes per row, eight rows per store instruction) instead of
// 32 pieces of 16 bytes per instruction: the fragmented form takes four times the store requests.  `stage`: 64 rows x 72
// halfs of LDS owned by this wavefront (row stride 144 bytes: 16-byte aligned pieces, rows spread over the banks).  Whole tiles only.
template <int ACT>
__device__ __forceinline__ void gated_store_lines(const BigArgs& a, floatx16 (&acc)[4][2], int nt_first, long row_first, int lane, half_t* stage,
                                                  const float (&rinv2)[2]) {
    constexpr int LDSROW = 72;
    const int lh = lane >> 5, r = lane & 31;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        float b1[8], b2[8];
#pragma unroll
        for (int v = 0; v < 8; ++v) {
            const int f = (nt_first + j) * 16 + 8 * (v / 4) + 4 * lh + (v % 4);
            b1[v] = a.bias[f]; b2[v] = a.bias2[f];
        }
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
            for (int g = 0; g < 2; ++g) {
                half4v o;
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = (half_t)(act_apply_c<ACT>(acc[j][i][4 * g + e] * rinv2[i] + b1[4 * g + e]) * (acc[j][i][4 * g + e + 8] * rinv2[i] + b2[4 * g + e]));
                *(half4v*)(stage + (32 * i + r) * LDSROW + 16 * j + 8 * g + 4 * lh) = o;
            }
        }
    }
    __builtin_amdgcn_wave_barrier();
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    const int piece = lane & 7, rr = lane >> 3;
    half8 line[8];
#pragma unroll
    for (int ps = 0; ps < 8; ++ps) line[ps] = *(const half8*)(stage + (8 * ps + rr) * LDSROW + 8 * piece);
#pragma unroll
    for (int ps = 0; ps < 8; ++ps) *(half8*)(a.out16 + (row_first + 8 * ps + rr) * a.ld16 + (long)nt_first * 16 + 8 * piece) = line[ps];
}

// The same for one 32-column tile of a residual projection (64 rows x 32 fp32 columns = one 128-byte line per row): the
// old residual values are requested in line layout first, the accumulators cross through LDS (64 rows x 36 floats), and
// x, half(gamma x) and the tile's sums of squares leave from the line layout (a row's 32 columns sit in eight lanes).
// Same arithmetic per element as the direct form (acc * rinv + bias, then + old); the sums of squares add in another order.
template <bool RESID>     // false: plain fp32 output with bias (no old values, no fp16 copy)
__device__ __forceinline__ void resid_store_lines(const BigArgs& a, const floatx16 (&acc2)[2], int nt, long row_first, int lane, float* stage,
                                                  const float (&rinv2)[2]) {
    constexpr int LDSROW = 36;
    const int lh = lane >> 5, r = lane & 31, piece = lane & 7, rr = lane >> 3;
    floatx4 old[8];
#pragma unroll
    // (the old values were written a whole GEMM ago and are read once here; the new ones are read a whole GEMM from now)
    for (int ps = 0; ps < 8; ++ps) old[ps] = RESID ? load_once((const floatx4*)(a.out + (row_first + 8 * ps + rr) * a.ld_out + (long)nt * 32 + 4 * piece)) : floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    float bb[16];
#pragma unroll
    for (int v = 0; v < 16; ++v) bb[v] = a.bias[nt * 32 + 8 * (v / 4) + 4 * lh + (v % 4)];
    const floatx4 gm = (RESID && a.xg16) ? *(const floatx4*)(a.gamma + nt * 32 + 4 * piece) : floatx4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            floatx4 sv;
#pragma unroll
            for (int e = 0; e < 4; ++e) sv[e] = acc2[i][4 * g + e] * rinv2[i] + bb[4 * g + e];
            *(floatx4*)(stage + (32 * i + r) * LDSROW + 8 * g + 4 * lh) = sv;
        }
    __builtin_amdgcn_wave_barrier();
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    floatx4 v[8];
#pragma unroll
    for (int ps = 0; ps < 8; ++ps) v[ps] = *(const floatx4*)(stage + (8 * ps + rr) * LDSROW + 4 * piece);
#pragma unroll
    for (int ps = 0; ps < 8; ++ps) {
        const long row = row_first + 8 * ps + rr;
        floatx4 sv;
#pragma unroll
        for (int e = 0; e < 4; ++e) sv[e] = RESID ? v[ps][e] + old[ps][e] : v[ps][e];
        __builtin_nontemporal_store(sv, (floatx4*)(a.out + row * a.ld_out + (long)nt * 32 + 4 * piece));
        if (RESID && a.xg16) {
            half4v xg;
            float q = 0.0f;
#pragma unroll
            for (int e = 0; e < 4; ++e) { xg[e] = (half_t)(gm[e] * sv[e]); q += sv[e] * sv[e]; }
            *(half4v*)(a.xg16 + row * a.ld_xg + (long)nt * 32 + 4 * piece) = xg;
            q += __shfl_xor(q, 1, 64);
            q += __shfl_xor(q, 2, 64);
            q += __shfl_xor(q, 4, 64);
            if (piece == 0) a.ssq_out[(long)nt * a.ssq_ld + row] = q;
        }
    }
    __builtin_amdgcn_wave_barrier();          // the next tile's accumulators overwrite the stage
}

// Ungated activation output (ReLU / SiLU / LeakyReLU feed-forward, MoE experts): a wavefront's 64 rows x 128 columns go
// out in two halves of 64 columns (one 128-byte line per row each) through the same 64 x 72 halfs of LDS.
template <int ACT>
__device__ __forceinline__ void act_store_lines(const BigArgs& a, floatx16 (&acc)[4][2], int nt_first, long row_first, int lane, half_t* stage,
                                                const float (&rinv2)[2]) {
    constexpr int LDSROW = 72;
    const int lh = lane >> 5, r = lane & 31, piece = lane & 7, rr = lane >> 3;
#pragma unroll
    for (int hj = 0; hj < 2; ++hj) {
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) {
            const int j = 2 * hj + jj;
            float bb[16];
#pragma unroll
            for (int v = 0; v < 16; ++v) bb[v] = a.bias[(nt_first + j) * 32 + 8 * (v / 4) + 4 * lh + (v % 4)];
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    half4v o;
#pragma unroll
                    for (int e = 0; e < 4; ++e) o[e] = (half_t)act_apply_c<ACT>(acc[j][i][4 * g + e] * rinv2[i] + bb[4 * g + e]);
                    *(half4v*)(stage + (32 * i + r) * LDSROW + 32 * jj + 8 * g + 4 * lh) = o;
                }
        }
        __builtin_amdgcn_wave_barrier();
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        half8 line[8];
#pragma unroll
        for (int ps = 0; ps < 8; ++ps) line[ps] = *(const half8*)(stage + (8 * ps + rr) * LDSROW + 8 * piece);
#pragma unroll
        for (int ps = 0; ps < 8; ++ps) *(half8*)(a.out16 + (row_first + 8 * ps + rr) * a.ld16 + (long)(nt_first + 2 * hj) * 32 + 8 * piece) = line[ps];
        __builtin_amdgcn_wave_barrier();          // the second half overwrites the stage
    }
}

// Keys or values of one wavefront of a QKV projection (64 rows = two 32-position chunks, 128 columns) into the
// fragment-major fp16 cache, in two passes of 64 columns through the wavefront's 64 x 72 halfs of LDS: the accumulators
// go in row-major (keys rotated first: a lane holds both elements of a pair), whole fragments come out, 16 bytes per lane
// and 1 KiB per store instruction.  Key fragment (tile, kd) of a chunk: lane (r, qq) holds position 8 (r / 4) + 4 tile +
// r % 4, elements 32 kd + 8 qq .. + 7; value fragment dt: lane (r, qq) holds element 16 dt + r at positions 8 qq .. + 7
// (the layouts kv_write_frag_kernel writes).  Same arithmetic per element as the unfused path: acc * rinv + bias, rotation
// with two roundings per output, one rounding to fp16.
template <int D, bool IS_K>
__device__ __forceinline__ void kv_store_frags(const BigArgs& a, floatx16 (&acc)[4][2], int nt_first, long row_first, int lane, half_t* stage,
                                               const float (&rinv2)[2]) {
    constexpr int LDSROW = 72, KD = D / 32;
    const int lh = lane >> 5, r = lane & 31, r16 = lane & 15, qq = lane >> 4;
    const int rel0 = nt_first * 32 - a.kv_col0 - (IS_K ? 0 : a.kv_gd);        // first column within the key (value) block
    long cbase[2]; int pos[2]; bool rows_ok[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const long row = row_first + 32 * i;
        rows_ok[i] = row < a.R;
        const long rc = rows_ok[i] ? row : 0;
        const int bq = (int)(rc / a.kv_Tq), tq = (int)(rc % a.kv_Tq);
        pos[i] = a.kv_pos0 + tq + r;
        cbase[i] = (long)bq * a.kv_hkv * a.kv_max_len * D + (long)((a.kv_pos0 + tq) >> 5) * (32 * D);
    }
#pragma unroll
    for (int cg = 0; cg < 2; ++cg) {
        const int relc = rel0 + 64 * cg, kvh = relc / D, dofs = relc % D;
        floatx4 bb[2][4]; floatx2 cs[2][2][4], sn[2][2][4];
#pragma unroll
        for (int jj = 0; jj < 2; ++jj)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                bb[jj][g] = *(const floatx4*)(a.bias + (nt_first + 2 * cg + jj) * 32 + 8 * g + 4 * lh);
                if (IS_K && a.rope_cos) {
#pragma unroll
                    for (int i = 0; i < 2; ++i) {
                        const long ro = (long)pos[i] * (D / 2) + (dofs + 32 * jj + 8 * g + 4 * lh) / 2;
                        cs[i][jj][g] = *(const floatx2*)(a.rope_cos + ro); sn[i][jj][g] = *(const floatx2*)(a.rope_sin + ro);
                    }
                }
            }
#pragma unroll
        for (int jj = 0; jj < 2; ++jj)
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    float x[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) x[e] = acc[2 * cg + jj][i][4 * g + e] * rinv2[i] + bb[jj][g][e];
                    half4v o;
                    if (IS_K && a.rope_cos) {
#pragma unroll
                        for (int pr = 0; pr < 2; ++pr) {
                            float y0, y1;
                            rope_pair(x[2 * pr], x[2 * pr + 1], cs[i][jj][g][pr], sn[i][jj][g][pr], y0, y1);
                            o[2 * pr] = (half_t)y0; o[2 * pr + 1] = (half_t)y1;
                        }
                    } else {
                        // (the fp32 value is rounded before the conversion, as it is when the projection's output passes
                        // through memory: a multiply-add fused with the conversion rounds once and differs in one of 2^13 cases)
#pragma unroll
                        for (int e = 0; e < 4; ++e) { float xe = x[e]; asm volatile("" : "+v"(xe)); o[e] = (half_t)xe; }
                    }
                    *(half4v*)(stage + (32 * i + r) * LDSROW + 32 * jj + 8 * g + 4 * lh) = o;
                }
        __builtin_amdgcn_wave_barrier();
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (IS_K) {
            half8 fr[2][2][2];
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int tile = 0; tile < 2; ++tile)
#pragma unroll
                    for (int kdl = 0; kdl < 2; ++kdl)
                        fr[i][tile][kdl] = *(const half8*)(stage + (32 * i + 8 * (r16 >> 2) + 4 * tile + (r16 & 3)) * LDSROW + 32 * kdl + 8 * qq);
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                if (!rows_ok[i]) continue;
                half_t* dst = a.kcache + cbase[i] + (long)kvh * a.kv_max_len * D + lane * 8;
#pragma unroll
                for (int tile = 0; tile < 2; ++tile)
#pragma unroll
                    for (int kdl = 0; kdl < 2; ++kdl) *(half8*)(dst + (tile * KD + dofs / 32 + kdl) * 512) = fr[i][tile][kdl];
            }
        } else {
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                half8 fr[4];
#pragma unroll
                for (int dtl = 0; dtl < 4; ++dtl)
#pragma unroll
                    for (int jx = 0; jx < 8; ++jx) fr[dtl][jx] = stage[(32 * i + 8 * qq + jx) * LDSROW + 16 * dtl + r16];
                if (!rows_ok[i]) continue;
                half_t* dst = a.vcache + cbase[i] + (long)kvh * a.kv_max_len * D + lane * 8;
#pragma unroll
                for (int dtl = 0; dtl < 4; ++dtl) *(half8*)(dst + (dofs / 16 + dtl) * 512) = fr[dtl];
            }
        }
        __builtin_amdgcn_wave_barrier();          // the second pass overwrites the stage
    }
}

template <int EPI, int NI = 4>      // NI: 32-row tiles per wavefront (the wavefront's rows start at 32 NI wr)
__device__ __forceinline__ void big_gemm_store(const BigArgs& a, floatx16 (&acc)[4][NI], int nt0, long row0, int wr, int wn, int lane, half_t* stage = nullptr) {
    // accumulator (j, i), lane l, register v = 4 g + e: column (nt0 + 4 wn + j) * 32 + 8 g + 4 (l / 32) + e,
    // row row0 + 128 wr + 32 i + l % 32.  Biases (and the residual) are fetched in batches before the first store
    // of a column tile, and the four consecutive columns of a group go out as one 16-byte (fp32) or 8-byte (fp16) store.
    const int lh = lane >> 5;
    const bool vec_ok = (a.n_valid % 4 == 0) && ((EPI == BEPI_ACT16 ? a.ld16 : a.ld_out) % 4 == 0);
    float rinv4[NI];          // deferred norm: scale of this lane's four rows (1 when the input is already normalised)
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        const long row = row0 + 32 * NI * wr + 32 * i + (lane & 31);
        rinv4[i] = (a.rinv && row < a.R) ? a.rinv[row] : 1.0f;
    }
    if constexpr (EPI == BEPI_ACT16 && NI == 2) {
        // whole 64 x 64 output block of a gated projection with 16-byte aligned rows: line stores through LDS
        const long rf = row0 + 64 * wr;
        const int ntf = nt0 + 4 * wn;
        if (stage && a.gated && rf + 64 <= a.R && ntf + 4 <= a.NT && (ntf + 4) * 16 <= a.n_valid && (a.ld16 & 7) == 0) {
            const float r2[2] = {rinv4[0], rinv4[1]};
            with_act(a.act, [&](auto A) { gated_store_lines<decltype(A)::value>(a, acc, ntf, rf, lane, stage, r2); });
            return;
        }
        if (stage && !a.gated && rf + 64 <= a.R && ntf + 4 <= a.NT && (ntf + 4) * 32 <= a.n_valid && (a.ld16 & 7) == 0) {
            const float r2[2] = {rinv4[0], rinv4[1]};
            with_act(a.act, [&](auto A) { act_store_lines<decltype(A)::value>(a, acc, ntf, rf, lane, stage, r2); });
            return;
        }
    }
    if constexpr ((EPI == BEPI_RESID || EPI == BEPI_F32_BIAS) && NI == 2) {
        const long rf = row0 + 64 * wr;
        const int ntf = nt0 + 4 * wn;
        constexpr bool RS = EPI == BEPI_RESID;
        if constexpr (!RS) {
            // key and value columns of a QKV projection that writes the cache itself (whole wavefronts: the column counts
            // are multiples of 128, the launch code checks the rest)
            if (stage && a.kcache && ntf * 32 >= a.kv_col0) {
                if (ntf >= a.NT) return;
                const float r2[2] = {rinv4[0], rinv4[1]};
                const bool is_k = ntf * 32 < a.kv_col0 + a.kv_gd;
                if (a.kv_D == 64) { if (is_k) kv_store_frags<64, true>(a, acc, ntf, rf, lane, stage, r2); else kv_store_frags<64, false>(a, acc, ntf, rf, lane, stage, r2); }
                else { if (is_k) kv_store_frags<128, true>(a, acc, ntf, rf, lane, stage, r2); else kv_store_frags<128, false>(a, acc, ntf, rf, lane, stage, r2); }
                return;
            }
        }
        if (stage && rf + 64 <= a.R && ntf + 4 <= a.NT && (ntf + 4) * 32 <= a.n_valid && (a.ld_out & 3) == 0 && (!RS || !a.xg16 || (a.ld_xg & 3) == 0)) {
            const float r2[2] = {rinv4[0], rinv4[1]};
            resid_store_lines<RS>(a, acc[0], ntf + 0, rf, lane, (float*)stage, r2);
            resid_store_lines<RS>(a, acc[1], ntf + 1, rf, lane, (float*)stage, r2);
            resid_store_lines<RS>(a, acc[2], ntf + 2, rf, lane, (float*)stage, r2);
            resid_store_lines<RS>(a, acc[3], ntf + 3, rf, lane, (float*)stage, r2);
            return;
        }
    }
    // one column tile per call with a compile-time tile number: the accumulators must only ever be indexed statically
    auto tile_out = [&](auto J) {
        constexpr int j = decltype(J)::value;
        const int nt = nt0 + 4 * wn + j;
        if (nt >= a.NT) return;
        if (EPI == BEPI_ACT16 && a.gated) {
            float b1[8], b2[8];
#pragma unroll
            for (int v = 0; v < 8; ++v) {
                const int f = nt * 16 + 8 * (v / 4) + 4 * lh + (v % 4);
                b1[v] = f < a.n_valid ? a.bias[f] : 0.0f;
                b2[v] = f < a.n_valid ? a.bias2[f] : 0.0f;
            }
#pragma unroll
            for (int i = 0; i < NI; ++i) {
                const long row = row0 + 32 * NI * wr + 32 * i + (lane & 31);
                if (row >= a.R) continue;
                const float rv = rinv4[i];
#pragma unroll
                for (int g = 0; g < 2; ++g) {
                    const int f0 = nt * 16 + 8 * g + 4 * lh;
                    half4v o;
#pragma unroll
                    for (int e = 0; e < 4; ++e) o[e] = (half_t)(act_apply(a.act, acc[j][i][4 * g + e] * rv + b1[4 * g + e]) * (acc[j][i][4 * g + e + 8] * rv + b2[4 * g + e]));
                    half_t* dst = a.out16 + row * a.ld16 + f0;
                    if (vec_ok && f0 + 3 < a.n_valid) *(half4v*)dst = o;
                    else {
#pragma unroll
                        for (int e = 0; e < 4; ++e) if (f0 + e < a.n_valid) dst[e] = o[e];
                    }
                }
            }
        } else {
            float bb[16];
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int col = nt * 32 + 8 * (v / 4) + 4 * lh + (v % 4);
                bb[v] = col < a.n_valid ? a.bias[col] : 0.0f;
            }
            float gm[16], rowsq[NI];
#pragma unroll
            for (int i = 0; i < NI; ++i) rowsq[i] = 0.0f;
            if (EPI == BEPI_RESID && a.xg16) {
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int col = nt * 32 + 8 * (v / 4) + 4 * lh + (v % 4);
                    gm[v] = col < a.n_valid ? a.gamma[col] : 0.0f;
                }
            }
            floatx4 old[NI][4];
            if (EPI == BEPI_RESID) {
#pragma unroll
                for (int i = 0; i < NI; ++i) {
                    const long row = row0 + 32 * NI * wr + 32 * i + (lane & 31);
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const int c0 = nt * 32 + 8 * g + 4 * lh;
                        const float* src = a.out + row * a.ld_out + c0;
                        if (row < a.R && vec_ok && c0 + 3 < a.n_valid) old[i][g] = *(const floatx4*)src;
                        else {
#pragma unroll
                            for (int e = 0; e < 4; ++e) old[i][g][e] = (row < a.R && c0 + e < a.n_valid) ? src[e] : 0.0f;
                        }
                    }
                }
            }
#pragma unroll
            for (int i = 0; i < NI; ++i) {
                const long row = row0 + 32 * NI * wr + 32 * i + (lane & 31);
                if (row >= a.R) continue;
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int c0 = nt * 32 + 8 * g + 4 * lh;
                    floatx4 s;
#pragma unroll
                    for (int e = 0; e < 4; ++e) s[e] = acc[j][i][4 * g + e] * rinv4[i] + bb[4 * g + e];
                    if (EPI == BEPI_ACT16) {
                        half4v o;
#pragma unroll
                        for (int e = 0; e < 4; ++e) o[e] = (half_t)act_apply(a.act, s[e]);
                        half_t* dst = a.out16 + row * a.ld16 + c0;
                        if (vec_ok && c0 + 3 < a.n_valid) *(half4v*)dst = o;
                        else {
#pragma unroll
                            for (int e = 0; e < 4; ++e) if (c0 + e < a.n_valid) dst[e] = o[e];
                        }
                    } else {
                        if (EPI == BEPI_RESID) {
#pragma unroll
                            for (int e = 0; e < 4; ++e) s[e] = s[e] + old[i][g][e];
                            if (a.xg16) {
                                half4v xg;
#pragma unroll
                                for (int e = 0; e < 4; ++e) {
                                    const bool ok = c0 + e < a.n_valid;
                                    xg[e] = (half_t)(ok ? gm[4 * g + e] * s[e] : 0.0f);
                                    rowsq[i] += ok ? s[e] * s[e] : 0.0f;
                                }
                                half_t* xd = a.xg16 + row * a.ld_xg + c0;
                                if (vec_ok && (a.ld_xg & 3) == 0 && c0 + 3 < a.n_valid) *(half4v*)xd = xg;
                                else {
#pragma unroll
                                    for (int e = 0; e < 4; ++e) if (c0 + e < a.n_valid) xd[e] = xg[e];
                                }
                            }
                        }
                        float* dst = a.out + row * a.ld_out + c0;
                        if (vec_ok && c0 + 3 < a.n_valid) *(floatx4*)dst = s;
                        else {
#pragma unroll
                            for (int e = 0; e < 4; ++e) if (c0 + e < a.n_valid) dst[e] = s[e];
                        }
                    }
                }
            }
            if (EPI == BEPI_RESID && a.xg16) {
                // the two lane halves hold the two column halves of a row's tile
#pragma unroll
                for (int i = 0; i < NI; ++i) {
                    const float q = rowsq[i] + __shfl_xor(rowsq[i], 32, 64);
                    const long row = row0 + 32 * NI * wr + 32 * i + (lane & 31);
                    if (lane < 32 && row < a.R) a.ssq_out[(long)nt * a.ssq_ld + row] = q;
                }
            }
        }
    };
    tile_out(std::integral_constant<int, 0>{});
    tile_out(std::integral_constant<int, 1>{});
    tile_out(std::integral_constant<int, 2>{});
    tile_out(std::integral_constant<int, 3>{});
}

// LDS-tiled prefill GEMM.  Block tile 256 rows x 256 columns, 4 wavefronts, each owning 128 x 128 (4 x 4 MFMA
// tiles of 32 x 32, 256 accumulator registers).  K advances in chunks of CK k-tiles (16 CK columns): per chunk the
// block stages 8 CK weight fragments (already fragment-ordered in memory: straight 1 KiB copies) and 8 CK activation
// fragments (row-major in memory, scattered into fragment order) in LDS, double buffered: the next chunk's global
// loads are in flight in registers while the MFMAs of the current chunk run, one barrier per chunk.
// Per k-tile a wavefront reads 8 fragments from LDS for 16 MFMAs.  Dynamic LDS: 2 x 16 KiB x CK.
template <int EPI, int CK>
__global__ __launch_bounds__(256) void big_gemm2_f16_kernel(BigArgs a) {
    extern __shared__ __attribute__((aligned(16))) half_t big_smem[];
    constexpr int FR = 8 * CK;                       // fragments of one operand per chunk
    constexpr int LPT = FR / 4;                      // 16-byte loads per thread per operand and chunk
    half_t* sW = big_smem;                           // [2][FR * 512]
    half_t* sX = big_smem + 2 * FR * 512;            // [2][FR * 512]
    const int t = threadIdx.x, lane = t & 63, w = __builtin_amdgcn_readfirstlane(t >> 6);
    const int wr = w >> 1, wn = w & 1;
    // Block -> tile: workgroups go to the 8 XCDs round robin (id % 8) and each XCD has its own L2, so the 32 blocks an
    // XCD runs at a time are laid out as one patch of 8 row tiles x 4 column tiles (12 distinct operand tiles for 32
    // blocks); consecutive patches go to different XCDs.
    const int CT = (a.NT + 7) / 8, RT = (int)((a.R + 255) / 256), PC = (CT + 3) / 4;
    const int xcd = blockIdx.x & 7, seq = blockIdx.x >> 3;
    const int patch = (seq >> 5) * 8 + xcd, q = seq & 31;
    const int ctile = (patch % PC) * 4 + (q & 3), rtile = (patch / PC) * 8 + (q >> 2);
    if (ctile >= CT || rtile >= RT) return;
    const int nt0 = ctile * 8;
    const long row0 = (long)rtile * 256;
    floatx16 acc[4][4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[j][i][v] = 0.0f;

    const half8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
    const int NC = (a.KT + CK - 1) / CK;
    half8 gw[LPT], gx[LPT];
    // fragment f of the chunk = (n-tile or row tile f / CK, k-tile f % CK); thread t fills lane t % 64 of fragments
    // t / 64 + 4 i of both operands, so every LDS store of a wavefront is one contiguous KiB (no bank conflicts); the
    // activation rows are read 16 bytes per lane (the neighbouring pieces of a row follow in the next k-tiles)
    auto gload = [&](int c) {
#pragma unroll
        for (int i = 0; i < LPT; ++i) {
            const int f = i * 4 + (t >> 6);
            const int nt = nt0 + f / CK, kt = c * CK + f % CK;
            gw[i] = (nt < a.NT && kt < a.KT) ? *(const half8*)(a.W + (((long)nt * a.KT + kt) * 64 + lane) * 8) : zero8;
            const int row = (f / CK) * 32 + (lane & 31), ktx = c * CK + f % CK;
            gx[i] = (row0 + row < a.R && ktx < a.KT) ? *(const half8*)(a.X + (row0 + row) * (long)a.ldx + ktx * 16 + 8 * (lane >> 5)) : zero8;
        }
    };
    auto lstore = [&](int buf) {
#pragma unroll
        for (int i = 0; i < LPT; ++i) {
            const int f = i * 4 + (t >> 6);
            *(half8*)(sW + ((long)buf * FR + f) * 512 + lane * 8) = gw[i];
            *(half8*)(sX + ((long)buf * FR + f) * 512 + lane * 8) = gx[i];
        }
    };
    gload(0);
    lstore(0);
    __syncthreads();
    for (int c = 0; c < NC; ++c) {
        const int buf = c & 1;
        if (c + 1 < NC) gload(c + 1);
        const half_t* bw = sW + (long)buf * FR * 512 + lane * 8;
        const half_t* bx = sX + (long)buf * FR * 512 + lane * 8;
        // fragments of k-tile kt + 1 are read from LDS while the 16 MFMAs of k-tile kt run
        half8 wfA[4], xfA[4], wfB[4], xfB[4];
        auto lread = [&](int kt, half8 (&wf)[4], half8 (&xf)[4]) {
#pragma unroll
            for (int j = 0; j < 4; ++j) wf[j] = *(const half8*)(bw + ((4 * wn + j) * CK + kt) * 512);
#pragma unroll
            for (int i = 0; i < 4; ++i) xf[i] = *(const half8*)(bx + ((4 * wr + i) * CK + kt) * 512);
        };
        auto mma = [&](half8 (&wf)[4], half8 (&xf)[4]) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf[j], xf[i], acc[j][i], 0, 0, 0);
        };
        // (the scheduling barriers keep the compiler from sinking the reads back to their first use)
        lread(0, wfA, xfA);
#pragma unroll
        for (int kt = 0; kt < CK; kt += 2) {
            if (kt + 1 < CK) lread(kt + 1, wfB, xfB);
            __builtin_amdgcn_sched_barrier(0);
            mma(wfA, xfA);
            __builtin_amdgcn_sched_barrier(0);
            if (kt + 1 < CK) {
                if (kt + 2 < CK) lread(kt + 2, wfA, xfA);
                __builtin_amdgcn_sched_barrier(0);
                mma(wfB, xfB);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        if (c + 1 < NC) lstore(buf ^ 1);
        __syncthreads();
    }
    big_gemm_store<EPI>(a, acc, nt0, row0, wr, wn, lane);
}

// 256 x 256 block tile with asynchronous staging: the operands go from global memory straight into LDS
// (global_load_lds_dwordx4: 64 lanes x 16 bytes land lane-linear, which is exactly a fragment), four stages of two
// k-tiles, so loads are issued three chunks ahead and need neither staging registers nor LDS stores.  The compiler
// cannot tell which LDS bytes an in-flight load will write and would wait for all of them before any LDS read, so the
// fragment reads and their waits are written out by hand.  Needs an even number of k-tiles; rows and column tiles
// beyond the matrix are clamped to the last valid one on load and dropped on store.
// Eight wavefronts, two per SIMD: wavefront (wr, wn) owns 64 rows x 128 columns (4 x 2 MFMA tiles of 32 x 32, 128
// accumulator registers).  Per k-tile a wavefront reads 4 weight and 2 activation fragments for 8 MFMAs.  The two
// wavefronts of a SIMD work half a period apart (see the loop): one reads fragments while the other multiplies.  With
// both in step (barrier, reads, products) all eight wavefronts read LDS at once while the matrix pipes idle, and then
// queue for the pipes: the gated up projection of 32 768 x 2048 x 11 264 took 1.21 ms that way against 1.07 ms.
// (Four wavefronts of 128 x 128 each, 16 fragment reads per 32 MFMAs and two thirds of the LDS traffic, measured
// slower still: the loop is bound by exposed waits, not by LDS bandwidth.)
__device__ __forceinline__ void lds_read_frags(unsigned wa, unsigned xa, half8 (&wf)[4], half8 (&xf)[2]) {
    asm volatile(
        "ds_read_b128 %0, %6\n\t"
        "ds_read_b128 %1, %6 offset:2048\n\t"
        "ds_read_b128 %2, %6 offset:4096\n\t"
        "ds_read_b128 %3, %6 offset:6144\n\t"
        "ds_read_b128 %4, %7\n\t"
        "ds_read_b128 %5, %7 offset:2048"
        : "=&v"(wf[0]), "=&v"(wf[1]), "=&v"(wf[2]), "=&v"(wf[3]), "=&v"(xf[0]), "=&v"(xf[1])
        : "v"(wa), "v"(xa)
        : "memory");
}
template <int N>
__device__ __forceinline__ void lds_wait_frags(half8 (&wf)[4], half8 (&xf)[2]) {
    asm volatile("s_waitcnt lgkmcnt(%6)"
                 : "+v"(wf[0]), "+v"(wf[1]), "+v"(wf[2]), "+v"(wf[3]), "+v"(xf[0]), "+v"(xf[1])
                 : "n"(N)
                 : "memory");
}

template <int EPI>
__global__ __launch_bounds__(512) void big_gemm3_f16_kernel(BigArgs a) {
    extern __shared__ __attribute__((aligned(16))) half_t big_smem[];
    constexpr int CK = 2, NST = 4, FR = 8 * CK, PF = NST - 1;          // k-tiles per stage, stages, fragments per operand and stage, chunks requested ahead
    constexpr int STAGE = 2 * FR * 512;                  // halfs per stage: weight fragments, then activation fragments
    const int t = threadIdx.x, lane = t & 63, w = __builtin_amdgcn_readfirstlane(t >> 6);
    const int wr = w >> 1, wn = w & 1;                   // 4 x 2 wavefronts
    unsigned bid = blockIdx.x;
    int rot = 0;
    auto take_problem = [&](int e) {
        a.R = a.rows_tab[e]; a.W = a.Wtab[e]; a.X += e * a.x_estride;
        if (a.out) a.out += e * a.out_estride;
        if (a.out16) a.out16 += e * a.out16_estride;
        if (a.row_idx) a.row_idx += e * a.idx_estride;
    };
    if (a.blocks_per_problem && !a.packed_problems) {
        const int e = (int)(bid / (unsigned)a.blocks_per_problem);
        bid -= (unsigned)e * (unsigned)a.blocks_per_problem;
        take_problem(e);
        rot = e;      // a problem with fewer than eight patches would leave XCDs idle: problem e starts on XCD e % 8
    }
    const int CT = (a.NT + 7) / 8, PC = (CT + 3) / 4;
    const int RT = a.packed_problems ? a.packed_rt : (int)((a.R + 255) / 256);
    const int xcd = (int)((bid - (unsigned)rot) & 7), seq = (int)(bid >> 3);
    const int PH = a.patch_rows ? a.patch_rows : 8;          // a patch: PH row tiles x 4 column tiles
    const int patch = (seq / (4 * PH)) * 8 + xcd, q = seq % (4 * PH);
    const int ctile = (patch % PC) * 4 + (q & 3);
    int rtile = (patch / PC) * PH + (q >> 2);
    if (ctile >= CT || rtile >= RT) return;
    if (a.packed_problems) {
        // the problem whose tiles hold packed row tile `rtile` (block-uniform: the counts sit in scalar registers)
        int e = -1, first = 0;
        for (int i = 0; i < a.packed_problems; ++i) {
            const int tiles = (a.rows_tab[i] + 255) / 256;
            if (e < 0 && rtile < first + tiles) { e = i; rtile -= first; }
            first += tiles;
        }
        if (e < 0) return;
        take_problem(e);
    }
    const int nt0 = ctile * 8;
    const long row0 = (long)rtile * 256;
    floatx16 acc[4][2];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[j][i][v] = 0.0f;

    // wavefront w stages fragments f = 8 i + w (i = 0, 1; f / 2: n-tile or 16-row block, f % 2: k-tile) of both operands.
    // Activations: 1 KiB block f holds 16 rows x 64 bytes (both k-tiles of the chunk); lane l fetches 16-byte piece
    // s = (l % 4) ^ ((row / 4) % 4) of row 16 f + l / 4, so that four lanes read one contiguous 64-byte run and the
    // fragment reads below (32 rows x 2 pieces) spread evenly over the LDS banks
    const half_t* wsrc[2]; const half_t* xsrc[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int f = i * 8 + w, tl = f >> 1, ktl = f & 1;
        const int nt = min(nt0 + tl, a.NT - 1);
        wsrc[i] = a.W + (((long)nt * a.KT + ktl) * 64 + lane) * 8;
        const int rl = f * 16 + (lane >> 2);
        long row = min(row0 + rl, (long)a.R - 1);
        if (a.row_idx) row = a.row_idx[row];
        xsrc[i] = a.X + row * (long)a.ldx + 8 * ((lane & 3) ^ ((rl >> 2) & 3));
    }
    typedef const void __attribute__((address_space(1)))* gptr_t;
    typedef void __attribute__((address_space(3)))* lptr_t;
    auto issue = [&](int c) {
        half_t* st = big_smem + (c % NST) * STAGE;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int f = i * 8 + w;
            __builtin_amdgcn_global_load_lds((gptr_t)(wsrc[i] + (long)c * (CK * 512)), (lptr_t)(st + f * 512), 16, 0, 0);
            __builtin_amdgcn_global_load_lds((gptr_t)(xsrc[i] + (long)c * (CK * 16)), (lptr_t)(st + (FR + f) * 512), 16, 0, 0);
        }
    };
    const int NC = a.KT / CK;
    const unsigned lds0 = (unsigned)(size_t)(lptr_t)big_smem;
    const unsigned woff = (unsigned)(((4 * wn) * CK) * 1024 + lane * 16);
    const int xr = 64 * wr + (lane & 31);
    const unsigned xsw = (unsigned)((xr >> 2) & 3);
    const unsigned xoff0 = (unsigned)(FR * 1024 + xr * 64 + 16 * (((lane >> 5)) ^ xsw));          // k-tile 0: s = l / 32
    const unsigned xoff1 = (unsigned)(FR * 1024 + xr * 64 + 16 * ((2 + (lane >> 5)) ^ xsw));      // k-tile 1: s = 2 + l / 32
    issue(0);
    if (NC > 1) issue(1);
    if (NC > 2) issue(2);
    // Two groups of four wavefronts (one per SIMD each; wavefronts w and w + 4 share a SIMD: grouping by w % 2 instead
    // measured 30 % slower) run the same chunks half a period apart with one block barrier per chunk: behind barrier c
    // the first group reads its fragments of chunk c from LDS while the second multiplies chunk c - 1 out of its
    // registers, then the first multiplies chunk c while the second reads it.  Before barrier c every wavefront has
    // waited for its own part of chunk c and has read chunk c - 1, so the loads of chunk c + 3 may overwrite that stage.
    // Both groups pass the same number of barriers.
    const int g = w >> 2;
    half8 wfA[4], xfA[2], wfB[4], xfB[2];
    auto wait_loads = [&](int c) {          // this wavefront's part of chunk c + 1 has landed
        const int later = max(0, min(PF - 1, NC - 2 - c));
        if (later == 2) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
        else if (later == 1) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    };
    auto R = [&](int c, bool wait_now) {
        const unsigned sb = lds0 + (unsigned)((c % NST) * STAGE * 2);
        lds_read_frags(sb + woff, sb + xoff0, wfA, xfA);                   // k-tile 0
        lds_read_frags(sb + woff + 1024, sb + xoff1, wfB, xfB);            // k-tile 1
        if (c + PF < NC) issue(c + PF);
        if (wait_now) wait_loads(c);
        lds_wait_frags<0>(wfA, xfA);
        lds_wait_frags<0>(wfB, xfB);
        __builtin_amdgcn_sched_barrier(0);
    };
    auto M = [&]() {
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_setprio(1);
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int i = 0; i < 2; ++i) acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wfA[j], xfA[i], acc[j][i], 0, 0, 0);
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int i = 0; i < 2; ++i) acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wfB[j], xfB[i], acc[j][i], 0, 0, 0);
        __builtin_amdgcn_s_setprio(0);
        __builtin_amdgcn_sched_barrier(0);
    };
    wait_loads(-1);
    __builtin_amdgcn_s_barrier();                       // chunk 0 is in LDS
    if (g == 0) {
        for (int c = 0; c < NC; ++c) {
            if (c) { __builtin_amdgcn_s_barrier(); __builtin_amdgcn_sched_barrier(0); }
            R(c, false);
            M();
            wait_loads(c);          // (behind the products: half a period more for the loads than in front of them)
        }
    } else {
        R(0, true);
        for (int c = 1; c < NC; ++c) {
            __builtin_amdgcn_s_barrier();
            M();
            R(c, true);
        }
        M();
    }
    // (the first group is here while the second may still be reading the last chunk: the stages are dead, and each
    // wavefront owns 64 x 72 halfs of them for its epilogue, once every wavefront has passed this barrier)
    __builtin_amdgcn_s_barrier();
    big_gemm_store<EPI, 2>(a, acc, nt0, row0, wr, wn, lane, big_smem + w * (64 * 72));
}

// ------------------------------------------------------------------------------------------------
// fp32 GEMM (fp32 models: prefill and decode): C[ks][M][N] = A[M][K-range ks] * B[K-range][N], 64x64 tile,
// k accumulated sequentially inside a split.
// ------------------------------------------------------------------------------------------------
struct F32GemmArgs {
    const float* A; long lda; const float* B; long ldb; float* C; long ldc; long split_stride;
    int M, N, K, KS;
    const float* bias;     // optional, added when the result is final (KS == 1)
};

// The same product for up to 32 rows (decode steps of fp32 models): the weights are what costs, every element is read
// once, 16 bytes per thread.  Block = 64 columns x one K range (blockIdx.z of KS): thread (tx, ty) owns columns
// 4 tx .. 4 tx + 3 and the k = ty, ty + 16, ... of the range, with the rows' activations broadcast from LDS; the sixteen
// k-lanes are added in a fixed order (lanes 16 and 32 apart inside a wavefront, then the four wavefronts), so the result
// does not depend on scheduling.  Same split-K output convention as the kernel below.
template <int MR>      // rows held in registers: 8, 16 or 32
__global__ __launch_bounds__(256) void skinny_gemm_f32_kernel(F32GemmArgs a) {
    constexpr int KC = 8192 / MR;                       // k per staging pass: MR x KC floats = 32 KiB
    __shared__ float sX[MR * KC];
    __shared__ float red[4][MR][64];
    const int t = threadIdx.x, tx = t & 15, ty = t >> 4, lane = t & 63, w = t >> 6;
    const int col0 = blockIdx.x * 64 + tx * 4, ks = blockIdx.z;
    const int kper = (int)round_up(ceil_div(a.K, a.KS), 16);
    const int kb = ks * kper, ke = min(a.K, kb + kper);
    const bool vec = (a.ldb & 3) == 0 && col0 + 3 < a.N;
    float acc[MR][4];
#pragma unroll
    for (int m = 0; m < MR; ++m)
#pragma unroll
        for (int c = 0; c < 4; ++c) acc[m][c] = 0.0f;
    for (int k0 = kb; k0 < ke; k0 += KC) {
        const int kn = min(KC, ke - k0);
        __syncthreads();                                // the pass before is consumed
        for (int idx = t; idx < MR * kn; idx += 256) {
            const int m = idx / kn, k = idx - m * kn;
            sX[m * KC + k] = m < a.M ? a.A[(long)m * a.lda + k0 + k] : 0.0f;
        }
        __syncthreads();
        constexpr int U = MR <= 16 ? 8 : 4;             // weight rows in flight per thread
        for (int k = ty; k < kn; k += 16 * U) {
            floatx4 wv[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int kk = k + 16 * u;
                const float* src = a.B + (long)(k0 + kk) * a.ldb + col0;
                if (kk < kn && vec) wv[u] = load_once((const floatx4*)src);
                else {
#pragma unroll
                    for (int c = 0; c < 4; ++c) wv[u][c] = (kk < kn && col0 + c < a.N) ? src[c] : 0.0f;
                }
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int kk = k + 16 * u;
                if (kk >= kn) break;
#pragma unroll
                for (int m = 0; m < MR; ++m) {
                    const float xv = sX[m * KC + kk];
#pragma unroll
                    for (int c = 0; c < 4; ++c) acc[m][c] = fmaf(xv, wv[u][c], acc[m][c]);
                }
            }
        }
    }
    // k-lanes: ty = 4 w + (lane / 16): add the lanes 16 and 32 apart, then the wavefronts through LDS
#pragma unroll
    for (int m = 0; m < MR; ++m)
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            float v = acc[m][c];
            v += __shfl_xor(v, 16, 64);
            v += __shfl_xor(v, 32, 64);
            acc[m][c] = v;
        }
    if (lane < 16) {
#pragma unroll
        for (int m = 0; m < MR; ++m)
#pragma unroll
            for (int c = 0; c < 4; ++c) red[w][m][tx * 4 + c] = acc[m][c];
    }
    __syncthreads();
    for (int idx = t; idx < MR * 64; idx += 256) {
        const int m = idx >> 6, c = idx & 63, col = blockIdx.x * 64 + c;
        if (m < a.M && col < a.N) {
            float v = ((red[0][m][c] + red[1][m][c]) + red[2][m][c]) + red[3][m][c];
            if (a.bias) v += a.bias[col];
            a.C[ks * a.split_stride + (long)m * a.ldc + col] = v;
        }
    }
}

__global__ __launch_bounds__(256) void gemm_f32_kernel(F32GemmArgs a) {
    __shared__ float As[16][64 + 4];
    __shared__ float Bs[16][64 + 4];
    const int t = threadIdx.x, tx = t & 15, ty = t >> 4;
    const int col0 = blockIdx.x * 64, row0 = blockIdx.y * 64, ks = blockIdx.z;
    const int kper = (int)round_up(ceil_div(a.K, a.KS), 16);
    const int kb = ks * kper, ke = min(a.K, kb + kper);
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.0f;
    const int am = t >> 2, ak = (t & 3) * 4;
    const int bk = t >> 4, bn = (t & 15) * 4;
    for (int k0 = kb; k0 < ke; k0 += 16) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            int r = row0 + am, k = k0 + ak + j;
            As[ak + j][am] = (r < a.M && k < ke) ? a.A[(long)r * a.lda + k] : 0.0f;
            int kk = k0 + bk, c = col0 + bn + j;
            Bs[bk][bn + j] = (kk < ke && c < a.N) ? a.B[(long)kk * a.ldb + c] : 0.0f;
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
    float* C = a.C + ks * a.split_stride;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        int r = row0 + ty * 4 + i;
        if (r >= a.M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            int c = col0 + tx * 4 + j;
            if (c < a.N) C[(long)r * a.ldc + c] = a.bias ? acc[i][j] + a.bias[c] : acc[i][j];
        }
    }
}

// FFN activation for paths whose GEMM has no fused epilogue: out[r][f] = act(sum part[.][r][f] + b1[f])
// (* (sum part[.][r][F+f] + b3[f]) when gated)
template <typename AT>
__global__ void ffn_act_kernel(const float* __restrict__ part, int KS, long split_stride, long ldp, const float* __restrict__ b1,
                               const float* __restrict__ b3, int F, int gated, int act, AT* __restrict__ out, long ld_out, long R) {
    long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= R * F) return;
    long r = idx / F; int f = (int)(idx % F);
    // split-K partials in index order, eight requested at a time (unconditionally, the index clamped to the last split)
    auto sum_splits = [&](long off) {
        float acc = 0.0f;
        for (int k = 0; k < KS; k += 8) {
            float pk[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) pk[j] = part[min(k + j, KS - 1) * split_stride + off];
#pragma unroll
            for (int j = 0; j < 8; ++j) if (k + j < KS) acc += pk[j];
        }
        return acc;
    };
    float s = act_apply(act, sum_splits(r * ldp + f) + b1[f]);
    if (gated) s *= (sum_splits(r * ldp + F + f) + b3[f]);
    out[r * ld_out + f] = (AT)s;
}

// ------------------------------------------------------------------------------------------------
// residual update + normalisation, one block per row.
//   source   : embedding gather x = E[id] * scale  (TensorUtils.CreateTokensEmbeddings, Utils/TensorUtils.cs:147-156)
//              or x += (sum of split-K partials + bias)   (g.Affine then graph.Add with the layer input)
//              or x as it is
//   then RMSNorm (TensorApplyCPU.cs:1451-1496) or LayerNorm (:1360-1447) -> xn in the activation type.
// ------------------------------------------------------------------------------------------------
struct ResidNormArgs {
    float* x; long ldx; int h;
    const int* ids; const void* emb; int emb_f16; float emb_scale;
    // segment embeddings (TensorUtils.CreateTokensEmbeddings, Seq2SeqSharp/Utils/TensorUtils.cs:147-152): fp32 table
    // [segments][h], added to the scaled token embedding; seg_ids [rows] = segment of every row, null = segment 0
    const float* seg; const int* seg_ids;
    const float* part; int KS; long split_stride; long ld_part; const float* bias;
    const float* gamma; const float* beta; float eps; int norm_type;
    void* xn; long ldxn;
    int xn_kt;              // > 0 (fp16 only): xn is fragment packed with this many k-tiles; 0: row-major with ldxn
    const int* row_map;     // optional: block r works on row row_map[r] of x and writes row r of xn
    int* advance_pos;       // optional: block 0 increments this device counter (end of a decode step)
    // optional source: x += the MoE experts' outputs, each scaled by its router probability and added in expert order
    // (MoEFeedForward.cs:167-178; IndexSelectGrad, TensorApplyCPU.cs:1336-1356).  y[e][slot][col], slot[row * k + j] =
    // place of the row in the list of its j-th expert
    const float* moe_y; long moe_ldy; long moe_estride; const float* moe_probs; const float* moe_top; const int* moe_slot; int moe_k; int moe_E;
    int* moe_clear_counts;  // optional: block 0 clears the experts' row counters for the next router launch
};

template <typename AT, int NPT>   // NPT * 256 >= hidden
__global__ __launch_bounds__(256) void resid_norm_kernel(ResidNormArgs a) {
    __shared__ float sred[4];
    const int r = blockIdx.x, t = threadIdx.x;
    const long xr = a.row_map ? a.row_map[r] : r;
    const float* __restrict__ part = a.part;
    const float* __restrict__ xin = a.x + xr * a.ldx;
    float v[NPT];
    long erow = a.ids ? (long)a.ids[r] : 0;
    // all loads first (independent), then the arithmetic, then the stores; the MoE choices head the longest chain of
    // dependent loads (choice -> slot -> expert output), so they are requested before anything else
    constexpr int MAXK = 4;
    int te[MAXK], ts[MAXK];
#pragma unroll
    for (int j = 0; j < MAXK; ++j) {
        te[j] = (a.moe_y && j < a.moe_k && a.moe_k <= MAXK) ? (int)a.moe_top[xr * a.moe_k + j] : -1;
        ts[j] = (a.moe_y && j < a.moe_k && a.moe_k <= MAXK) ? a.moe_slot[xr * a.moe_k + j] : 0;
    }
    float gm[NPT], bt[NPT];
#pragma unroll
    for (int i = 0; i < NPT; ++i) {
        const int c = t + i * 256;
        gm[i] = (a.xn && c < a.h) ? a.gamma[c] : 0.0f;
        bt[i] = (a.xn && a.beta && c < a.h) ? a.beta[c] : 0.0f;
    }
#pragma unroll
    for (int i = 0; i < NPT; ++i) {
        int c = t + i * 256;
        v[i] = 0.0f;
        if (c < a.h) {
            if (a.ids) {
                float e = a.emb_f16 ? (float)((const half_t*)a.emb)[erow * a.h + c] : ((const float*)a.emb)[erow * a.h + c];
                v[i] = e * a.emb_scale;
                if (a.seg) v[i] = v[i] + a.seg[(long)(a.seg_ids ? a.seg_ids[r] : 0) * a.h + c];
            } else {
                v[i] = xin[c];
            }
        }
    }
    if (part) {
        float s[NPT];
#pragma unroll
        for (int i = 0; i < NPT; ++i) {
            int c = t + i * 256;
            s[i] = (c < a.h) ? part[(long)r * a.ld_part + c] : 0.0f;
        }
        // splits are added in index order; a batch of them is requested together (unconditionally, the index clamped to the
        // last split, so that the batch's loads are all in flight before the first is waited for)
        constexpr int GROUP = NPT <= 4 ? 8 : 4;
        for (int k = 1; k < a.KS; k += GROUP) {
            float p[GROUP][NPT];
#pragma unroll
            for (int j = 0; j < GROUP; ++j) {
                const int kk = min(k + j, a.KS - 1);
#pragma unroll
                for (int i = 0; i < NPT; ++i) {
                    const int c = min(t + i * 256, a.h - 1);
                    p[j][i] = part[kk * a.split_stride + (long)r * a.ld_part + c];
                }
            }
#pragma unroll
            for (int j = 0; j < GROUP; ++j) {
                if (k + j < a.KS) {
#pragma unroll
                    for (int i = 0; i < NPT; ++i) s[i] += p[j][i];
                }
            }
        }
#pragma unroll
        for (int i = 0; i < NPT; ++i) {
            int c = t + i * 256;
            if (c < a.h) v[i] = (s[i] + a.bias[c]) + v[i];
        }
    }
    if (a.moe_y) {
#pragma clang fp contract(off)
        if (a.moe_clear_counts && blockIdx.x == 0 && t < a.moe_E) a.moe_clear_counts[t] = 0;
        if (a.moe_k <= MAXK) {
            // the row's choices, their slots and probabilities once; then every expert output at once; added in expert order
            float tp[MAXK], yv[MAXK][NPT];
#pragma unroll
            for (int j = 0; j < MAXK; ++j) {
                tp[j] = te[j] >= 0 ? a.moe_probs[xr * a.moe_E + te[j]] : 0.0f;
#pragma unroll
                for (int i = 0; i < NPT; ++i) {
                    const int c = t + i * 256;
                    yv[j][i] = (te[j] >= 0 && c < a.h) ? a.moe_y[te[j] * a.moe_estride + (long)ts[j] * a.moe_ldy + c] : 0.0f;
                }
            }
            float out[NPT];
#pragma unroll
            for (int i = 0; i < NPT; ++i) out[i] = 0.0f;
            for (int e = 0; e < a.moe_E; ++e) {
#pragma unroll
                for (int j = 0; j < MAXK; ++j) {
                    if (te[j] == e) {
#pragma unroll
                        for (int i = 0; i < NPT; ++i) { const float sc = yv[j][i] * tp[j]; out[i] += sc; }
                    }
                }
            }
#pragma unroll
            for (int i = 0; i < NPT; ++i) v[i] = v[i] + out[i];
        } else {
            for (int i = 0; i < NPT; ++i) {
                const int c = t + i * 256;
                if (c >= a.h) continue;
                float out = 0.0f;
                for (int e = 0; e < a.moe_E; ++e)
                    for (int j = 0; j < a.moe_k; ++j)
                        if ((int)a.moe_top[xr * a.moe_k + j] == e) {
                            float sc = a.moe_y[e * a.moe_estride + (long)a.moe_slot[xr * a.moe_k + j] * a.moe_ldy + c] * a.moe_probs[xr * a.moe_E + e];
                            out += sc;
                        }
                v[i] = v[i] + out;
            }
        }
    }
    float sum = 0.0f, sq = 0.0f;
#pragma unroll
    for (int i = 0; i < NPT; ++i) {
        int c = t + i * 256;
        if (c < a.h) {
            if (a.ids || part || a.moe_y) a.x[xr * a.ldx + c] = v[i];
            sum += v[i]; sq += v[i] * v[i];
        }
    }
    if (a.advance_pos && r == 0 && t == 0) { a.advance_pos[0] += 1; a.advance_pos[1] += 1; }
    if (!a.xn) return;
    AT* out = (AT*)a.xn + (long)r * a.ldxn;
    if (a.norm_type == 0) {
        float tot = block_sum_256(sq, sred);
        float rms = sqrtf(tot / (float)a.h + a.eps);
#pragma unroll
        for (int i = 0; i < NPT; ++i) {
            int c = t + i * 256;
            if (c < a.h) {
                float y = gm[i] * (v[i] / rms);
                if (a.beta) y += bt[i];
                if (a.xn_kt > 0) ((AT*)a.xn)[xpack_index(r, c, a.xn_kt)] = (AT)y; else out[c] = (AT)y;
            }
        }
    } else {
        float mean = block_sum_256(sum, sred) / (float)a.h;
        float d2 = 0.0f;
#pragma unroll
        for (int i = 0; i < NPT; ++i) {
            int c = t + i * 256;
            if (c < a.h) { float d = v[i] - mean; d2 += d * d; }
        }
        float sigma = sqrtf(a.eps + block_sum_256(d2, sred) / (float)a.h);
#pragma unroll
        for (int i = 0; i < NPT; ++i) {
            int c = t + i * 256;
            if (c < a.h) {
                float y = gm[i] * ((v[i] - mean) / sigma);
                if (a.beta) y += bt[i];
                if (a.xn_kt > 0) ((AT*)a.xn)[xpack_index(r, c, a.xn_kt)] = (AT)y; else out[c] = (AT)y;
            }
        }
    }
}

// Residual tail for a split-K projection on the deferred-norm path: one block per 32-column tile.
// x[:, tile] += sum of the split-K partials (in split order) + bias; stores x, the next GEMM's packed input
// half(gamma * x) and the tile's per-row sum of squares.  All loads of a thread are issued before the first use.
struct ResidTailArgs {
    float* x; long ldx; int h; int rows;
    const float* part; int KS; long split_stride; long ld_part; const float* bias;
    const float* gamma; half_t* xg16; int xg_kt; float* ssq_out; int ssq_ld;
};
template <int RPT>      // rows per thread: 256 threads cover 8 rows x 32 columns per pass
__global__ __launch_bounds__(256) void resid_tail_kernel(ResidTailArgs a) {
    const int nt = blockIdx.x, t = threadIdx.x, n = t & 31, b0 = t >> 5;
    const int col = nt * 32 + n;
    const bool okc = col < a.h;
    float p[RPT][8], xv[RPT];
    const float bias = okc ? a.bias[col] : 0.0f, gm = okc ? a.gamma[col] : 0.0f;
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
        const int b = b0 + 8 * i;
        const bool ok = okc && b < a.rows;
        xv[i] = ok ? a.x[(long)b * a.ldx + col] : 0.0f;
#pragma unroll
        for (int k = 0; k < 8; ++k) p[i][k] = (ok && k < a.KS) ? a.part[k * a.split_stride + (long)b * a.ld_part + col] : 0.0f;
    }
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
        const int b = b0 + 8 * i;
        if (b >= a.rows) continue;                       // uniform over the 32 lanes that share a row
        float s = p[i][0];
#pragma unroll
        for (int k = 1; k < 8; ++k) if (k < a.KS) s += p[i][k];
        for (int k = 8; k < a.KS; ++k) s += a.part[k * a.split_stride + (long)b * a.ld_part + col];
        float v = 0.0f;
        if (okc) {
            v = (s + bias) + xv[i];
            a.x[(long)b * a.ldx + col] = v;
            a.xg16[xpack_index(b, col, a.xg_kt)] = (half_t)(gm * v);
        }
        float q = v * v;
#pragma unroll
        for (int o = 16; o > 0; o >>= 1) q += __shfl_xor(q, o, 64);
        if (n == 0) a.ssq_out[(long)nt * a.ssq_ld + b] = q;
    }
}

// 1 / rms of every row from the per-tile sums of squares (deferred RMSNorm, prefill): one thread per row
__global__ __launch_bounds__(256) void rinv_rows_kernel(const float* __restrict__ ssq, int ntiles, long ld, float inv_h, float eps,
                                                        float* __restrict__ rinv, long rows) {
    const long r = (long)blockIdx.x * 256 + threadIdx.x;
    if (r >= rows) return;
    float s = 0.0f;
    for (int t0 = 0; t0 < ntiles; t0 += 8) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = t0 + u < ntiles ? ssq[(long)(t0 + u) * ld + r] : 0.0f;
#pragma unroll
        for (int u = 0; u < 8; ++u) s += v[u];
    }
    rinv[r] = 1.0f / sqrtf(s * inv_h + eps);
}

// Deferred-norm entry: x = E[id] * scale (or x = row row_map[r] of an existing stream) -> the next GEMM's packed
// input half(gamma * x) and the per-column-tile sums of squares.  One block per row.
struct FnPrepArgs {
    float* x; long ldx; int h;
    const int* ids; const void* emb; int emb_f16; float emb_scale;
    const float* seg; const int* seg_ids;      // segment embeddings, as in ResidNormArgs
    const float* src; long ld_src; const int* row_map;
    const float* gamma; half_t* xg16; int xg_kt; float* ssq_out; long ssq_ld;
    long xg_ld;             // xg_kt == 0: xg16 is row-major with this leading dimension
    int ln;                 // deferred LayerNorm: also store the tiles' plain sums, behind the ceil(h / 32) tiles of sums of squares
};
// (row r of the launch; erow: embedding row when a.ids is set; NT threads, NPT elements each)
template <int NPT, int NT>
__device__ __forceinline__ void fn_prepare_row(const FnPrepArgs& a, int r, long erow, int t) {
    const long srow = a.row_map ? a.row_map[r] : r;
    // all requests first (unconditional, the column clamped), then the arithmetic and the stores
    float vin[NPT], gmv[NPT], sgv[NPT];
    const long seg_row = (a.ids && a.seg && a.seg_ids) ? a.seg_ids[r] : 0;
#pragma unroll
    for (int i = 0; i < NPT; ++i) {
        const int c = min(t + i * NT, a.h - 1);
        if (a.ids) vin[i] = a.emb_f16 ? (float)((const half_t*)a.emb)[erow * a.h + c] : ((const float*)a.emb)[erow * a.h + c];
        else vin[i] = a.src[srow * a.ld_src + c];
        gmv[i] = a.gamma[c];
        sgv[i] = (a.ids && a.seg) ? a.seg[seg_row * a.h + c] : 0.0f;
    }
#pragma unroll
    for (int i = 0; i < NPT; ++i) {
        const int c = t + i * NT;
        float v = 0.0f;
        if (c < a.h) {
            v = a.ids ? vin[i] * a.emb_scale : vin[i];
            if (a.ids && a.seg) v = v + sgv[i];
            a.x[(long)r * a.ldx + c] = v;
            if (a.xg_kt > 0) a.xg16[xpack_index(r, c, a.xg_kt)] = (half_t)(gmv[i] * v);
            else a.xg16[(long)r * a.xg_ld + c] = (half_t)(gmv[i] * v);
        }
        float q = v * v;
#pragma unroll
        for (int o = 16; o > 0; o >>= 1) q += __shfl_xor(q, o, 64);
        if ((t & 31) == 0 && c < a.h) a.ssq_out[(long)(c >> 5) * a.ssq_ld + r] = q;
        if (a.ln) {
            float sv = v;
#pragma unroll
            for (int o = 16; o > 0; o >>= 1) sv += __shfl_xor(sv, o, 64);
            if ((t & 31) == 0 && c < a.h) a.ssq_out[(long)(((a.h + 31) >> 5) + (c >> 5)) * a.ssq_ld + r] = sv;
        }
    }
}
template <int NPT>
__global__ __launch_bounds__(256) void fn_prepare_kernel(FnPrepArgs a) {
    const int r = blockIdx.x;
    fn_prepare_row<NPT, 256>(a, r, a.ids ? (long)a.ids[r] : 0, threadIdx.x);
}

// ------------------------------------------------------------------------------------------------
// attention
// ------------------------------------------------------------------------------------------------
struct AttnArgs {
    // q/k/v source: fp32 [KS][rows][ldq] partial sums + bias; columns: H*D queries, then Hkv*D keys, then Hkv*D values
    const float* qkv; int KS; long split_stride; long ldq; const float* bias;
    int H, Hkv;
    void* kcache; void* vcache; long max_len;      // [batch][Hkv][max_len][D]
    const float* rope_cos; const float* rope_sin;  // [max_len][D/2]; null = no rotary embedding
    const int* d_pos;                              // decode: number of cached positions, read on the device
    int pos0;                                      // prefill: cache offset of the first query row
    int Tq;                                        // prefill: query rows per sequence
    void* out; long ld_out;                        // [rows][H*D] in the activation type
    int out_kt;                                    // > 0: out is fragment packed with this many k-tiles
    float scale;
    const float* ssq; int ssq_nt; int ssq_ld; float inv_h; float eps;   // deferred RMSNorm of the projection input (see SkinnyArgs)
    int ln;      // deferred LayerNorm (see SkinnyArgs): plain sums behind the sums of squares, `bias` holds d[ldq] followed by c[ldq]
    int vt;      // 1: keys and values are stored fragment-major (kfrag_index / vfrag_index) for the MFMA attention kernels
    // decode with several blocks per (row, KV head): their number, the exchange area [pairs][S][G D + 2 G] floats and one counter per pair
    int S; float* xchg; int* xcount;
    // prefill of sequences padded to one length (Decoder.cs:656, 687-690): original lengths [batch], null = none were padded.
    // Query row r of sequence b sees columns c <= r while r < lens[b] (BuildSelfTriMask, TensorApplyCPU.cs:1040-1065); a row
    // from lens[b] on has every column masked, which after the softmax means: it attends to ALL columns of the padded
    // sequence, with scores rounded to multiples of 2^-9 by the float32 addition of -30000.
    const int* lens;
    // More than eight query heads per KV head: the heads of a KV head are served in kv_sub groups of G (the kernels'
    // template argument) heads each, a block per group.  The grid then counts Hkv * kv_sub "KV heads"; block index v
    // takes query heads v G ... v G + G - 1 and the cache and projection columns of KV head v / kv_sub.  At decode every
    // group of a KV head appends the same new row (the same values to the same place).  0 or 1: one group.
    int kv_sub;
};

// Single-query attention of G query heads that share one KV head over T cached positions.
// Lanes are grouped LPR to a cache row (16-byte loads, head_dim contiguous); a wavefront covers RPW rows per
// load and keeps UR loads of keys and of values in flight, refilling each register as soon as it is consumed.
// Every lane group keeps its own online-softmax state over the rows it visits; the groups of a wavefront are
// merged with lane shuffles and the NW wavefronts through LDS.
// sQ: LDS [G][D] queries, already rotated and scaled.  Result (fp32) is written to sOut [G][D] in LDS.
// ONCE: the launch reads every cached row once (a decode step), see load_once; a prefill's blocks share them through L2.
template <typename CT, int D, int G, int NW, bool ONCE = false>
__device__ __forceinline__ void attn_core(const float* sQ, const CT* Kb, const CT* Vb, int T, float* sM, float* sL, float* sAcc,
                                          float* sOut, bool quant = false) {
    constexpr int EPL = 16 / (int)sizeof(CT);
    constexpr int LPR = D / EPL;
    constexpr int RPW = 64 / LPR;
    constexpr int UR = 4;
    constexpr int SWEEP = NW * RPW * UR;
    typedef CT vec_t __attribute__((ext_vector_type(EPL)));
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sub = lane % LPR, rg = lane / LPR;
    auto kv_load = [](const vec_t* p) { if constexpr (ONCE) return load_once(p); else return *p; };

    // fp16 cache: queries are kept as packed halves and the dot product uses v_dot2_f32_f16 (fp32 accumulate);
    // fp32 cache: plain fp32 multiply-add
    constexpr bool H16 = sizeof(CT) == 2;
    float q[H16 ? 1 : G][H16 ? 1 : EPL];
    half2v q2[H16 ? G : 1][H16 ? EPL / 2 : 1];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        if constexpr (H16) {
#pragma unroll
            for (int e = 0; e < EPL / 2; ++e) {
                q2[g][e][0] = (half_t)sQ[g * D + sub * EPL + 2 * e];
                q2[g][e][1] = (half_t)sQ[g * D + sub * EPL + 2 * e + 1];
            }
        } else {
#pragma unroll
            for (int e = 0; e < EPL; ++e) q[g][e] = sQ[g * D + sub * EPL + e];
        }
    }
    float m[G], l[G], acc[G][EPL];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        m[g] = -INFINITY; l[g] = 0.0f;
#pragma unroll
        for (int e = 0; e < EPL; ++e) acc[g][e] = 0.0f;
    }
    vec_t kv[UR], vv[UR];
    int tt[UR];
#pragma unroll
    for (int u = 0; u < UR; ++u) {
        tt[u] = (u * NW + wave) * RPW + rg;
#pragma unroll
        for (int e = 0; e < EPL; ++e) { kv[u][e] = (CT)0.0f; vv[u][e] = (CT)0.0f; }
        if (tt[u] < T) {
            kv[u] = kv_load((const vec_t*)(Kb + (long)tt[u] * D + sub * EPL));
            vv[u] = kv_load((const vec_t*)(Vb + (long)tt[u] * D + sub * EPL));
        }
    }
    for (int base = 0; base < T; base += SWEEP) {
#pragma unroll
        for (int u = 0; u < UR; ++u) {
            const bool ok = tt[u] < T;
            const vec_t kc = kv[u];
            float vf[EPL];
#pragma unroll
            for (int e = 0; e < EPL; ++e) vf[e] = (float)vv[u][e];
            tt[u] += SWEEP;
            if (tt[u] < T) {
                kv[u] = kv_load((const vec_t*)(Kb + (long)tt[u] * D + sub * EPL));
                vv[u] = kv_load((const vec_t*)(Vb + (long)tt[u] * D + sub * EPL));
            }
            float s[G];
#pragma unroll
            for (int g = 0; g < G; ++g) {
                float d = 0.0f;
                if constexpr (H16) {
#pragma unroll
                    for (int e = 0; e < EPL / 2; ++e) {
                        half2v kp; kp[0] = (half_t)kc[2 * e]; kp[1] = (half_t)kc[2 * e + 1];
                        d = __builtin_amdgcn_fdot2(q2[g][e], kp, d, false);
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < EPL; ++e) d = fmaf(q[g][e], (float)kc[e], d);
                }
#pragma unroll
                for (int o = LPR / 2; o > 0; o >>= 1) d += __shfl_xor(d, o, 64);
                s[g] = quant ? d + (-30000.0f) : d;      // (a fully masked row: the float32 addition of the mask value rounds the score)
            }
            if (ok) {
#pragma unroll
                for (int g = 0; g < G; ++g) {
                    float mn = fmaxf(m[g], s[g]);
                    float corr = __expf(m[g] - mn);
                    float p = __expf(s[g] - mn);
                    l[g] = l[g] * corr + p;
#pragma unroll
                    for (int e = 0; e < EPL; ++e) acc[g][e] = acc[g][e] * corr + p * vf[e];
                    m[g] = mn;
                }
            }
        }
    }
    // merge the row groups of this wavefront
#pragma unroll
    for (int o = LPR; o < 64; o <<= 1) {
#pragma unroll
        for (int g = 0; g < G; ++g) {
            float m2 = __shfl_xor(m[g], o, 64), l2 = __shfl_xor(l[g], o, 64);
            float M = fmaxf(m[g], m2);
            float w1 = (m[g] == M) ? 1.0f : __expf(m[g] - M);
            float w2 = (m2 == M) ? 1.0f : __expf(m2 - M);
            l[g] = l[g] * w1 + l2 * w2;
#pragma unroll
            for (int e = 0; e < EPL; ++e) acc[g][e] = acc[g][e] * w1 + __shfl_xor(acc[g][e], o, 64) * w2;
            m[g] = M;
        }
    }
    if (rg == 0) {
#pragma unroll
        for (int g = 0; g < G; ++g) {
            if (sub == 0) { sM[wave * G + g] = m[g]; sL[wave * G + g] = l[g]; }
#pragma unroll
            for (int e = 0; e < EPL; ++e) sAcc[(wave * G + g) * D + sub * EPL + e] = acc[g][e];
        }
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < G * D; idx += NW * 64) {
        int g = idx / D, d = idx % D;
        float M = -INFINITY;
        for (int i = 0; i < NW; ++i) M = fmaxf(M, sM[i * G + g]);
        float L = 0.0f, O = 0.0f;
        for (int i = 0; i < NW; ++i) {
            float wgt = __expf(sM[i * G + g] - M);    // wavefronts that saw no row have m = -inf -> weight 0
            L += sL[i * G + g] * wgt;
            O += sAcc[(i * G + g) * D + d] * wgt;
        }
        sOut[idx] = O / L;
    }
    __syncthreads();
}

template <typename CT, int D, int G, int NW>
struct AttnSmem {
    float in[(G + 2) * D];
    float q[G * D];
    float m[NW * G];
    float l[NW * G];
    float acc[NW * G * D];
    float out[G * D];
};

// decode step: grid (Hkv, batch).  Sums the QKV split-K partials, applies RoPE at position pos, appends the new
// key/value to the cache in place, then attends over pos+1 positions.
// Replaces: AsContiguous head split, RoPE, GQA Expand, Concate(cache), MulBatch, Softmax, MulBatch, transpose
// (Seq2SeqSharp/Layers/GroupQueryAttention.cs:121-224, Layers/MultiHeadAttention.cs:133-230).
template <typename CT, typename AT, int D, int G>
__global__ __launch_bounds__(1024) void attn_decode_kernel(AttnArgs a) {
    constexpr int NW = 16, NTH = NW * 64;
    __shared__ AttnSmem<CT, D, G, NW> sm;
    const int kvh = blockIdx.x, b = blockIdx.y, t = threadIdx.x;
    const int kvc = a.kv_sub > 1 ? kvh / a.kv_sub : kvh;       // the KV head whose cache this group of query heads reads
    const int pos = *a.d_pos;
    const int HD = a.H * D, GD = a.Hkv * D;
    float rinv = 1.0f, mean = 0.0f;
    if (a.ssq) {
        float s = 0.0f;
        for (int tt = (t & 63); tt < a.ssq_nt; tt += 64) s += a.ssq[(long)tt * a.ssq_ld + b];
        s = wave_sum(s);                                   // same butterfly in every wavefront: identical result
        if (a.ln) {
            float sv = 0.0f;
            for (int tt = (t & 63); tt < a.ssq_nt; tt += 64) sv += a.ssq[(long)(a.ssq_nt + tt) * a.ssq_ld + b];
            mean = wave_sum(sv) * a.inv_h;
            rinv = 1.0f / sqrtf(fmaxf(s * a.inv_h - mean * mean, 0.0f) + a.eps);
        } else {
            rinv = 1.0f / sqrtf(s * a.inv_h + a.eps);
        }
    }
    for (int idx = t; idx < (G + 2) * D; idx += NTH) {
        int col;
        if (idx < G * D) col = kvh * G * D + idx;
        else if (idx < (G + 1) * D) col = HD + kvc * D + (idx - G * D);
        else col = HD + GD + kvc * D + (idx - (G + 1) * D);
        // split-K partials in index order, eight requested at a time (unconditionally, the index clamped to the last split)
        float s = a.qkv[(long)b * a.ldq + col];
        for (int k = 1; k < a.KS; k += 8) {
            float pk[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) pk[j] = a.qkv[min(k + j, a.KS - 1) * a.split_stride + (long)b * a.ldq + col];
#pragma unroll
            for (int j = 0; j < 8; ++j) if (k + j < a.KS) s += pk[j];
        }
        sm.in[idx] = a.ln ? (s - mean * a.bias[a.ldq + col]) * rinv + a.bias[col] : s * rinv + a.bias[col];
    }
    __syncthreads();
    CT* Kb = (CT*)a.kcache + ((long)b * a.Hkv + kvc) * a.max_len * D;
    CT* Vb = (CT*)a.vcache + ((long)b * a.Hkv + kvc) * a.max_len * D;
    for (int p = t; p < (G + 1) * D / 2; p += NTH) {
        int vec = p / (D / 2), i = p % (D / 2);
        float x0 = sm.in[vec * D + 2 * i], x1 = sm.in[vec * D + 2 * i + 1], y0 = x0, y1 = x1;
        if (a.rope_cos) rope_pair(x0, x1, a.rope_cos[(long)pos * (D / 2) + i], a.rope_sin[(long)pos * (D / 2) + i], y0, y1);
        if (vec < G) { sm.q[vec * D + 2 * i] = a.scale * y0; sm.q[vec * D + 2 * i + 1] = a.scale * y1; }
        else { Kb[(long)pos * D + 2 * i] = (CT)y0; Kb[(long)pos * D + 2 * i + 1] = (CT)y1; }
    }
    for (int d = t; d < D; d += NTH) Vb[(long)pos * D + d] = (CT)sm.in[(G + 1) * D + d];
    __threadfence_block();
    __syncthreads();
    attn_core<CT, D, G, NW, true>(sm.q, Kb, Vb, pos + 1, sm.m, sm.l, sm.acc, sm.out);
    if (a.out_kt > 0) {
        for (int idx = t; idx < G * D; idx += NTH) ((AT*)a.out)[xpack_index(b, kvh * G * D + idx, a.out_kt)] = (AT)sm.out[idx];
    } else {
        AT* out = (AT*)a.out + (long)b * a.ld_out + kvh * G * D;
        for (int idx = t; idx < G * D; idx += NTH) out[idx] = (AT)sm.out[idx];
    }
}

// Fragment-major KV cache of the MFMA attention kernels (fp16, head_dim 64 or 128).  Positions are grouped in chunks
// of 32; within a chunk every 1 KiB block is exactly one A operand of v_mfma_f32_16x16x32_f16 (64 lanes x 8 halfs),
// so a wavefront's load instruction reads 1 KiB contiguous.
//   keys:   block (chunk, tile, kd), lane r + 16 qq holds K[t = 32 chunk + 8 (r / 4) + 4 tile + r % 4][d = 32 kd + 8 qq + j]
//   values: block (chunk, dt),       lane r + 16 qq holds V[t = 32 chunk + 8 qq + j][d = 16 dt + r]
__host__ __device__ inline long kfrag_index(int t, int d, int D) {
    const int c = t >> 5, tin = t & 31, q8 = tin >> 3, rem = tin & 7, tile = rem >> 2, r = 4 * q8 + (rem & 3);
    const int kd = d >> 5, qq = (d & 31) >> 3, j = d & 7;
    return ((((long)c * 2 + tile) * (D / 32) + kd) * 64 + r + 16 * qq) * 8 + j;
}
__host__ __device__ inline long vfrag_index(int t, int d, int D) {
    const int c = t >> 5, qq = (t & 31) >> 3, j = t & 7;
    return (((long)c * (D / 16) + (d >> 4)) * 64 + (d & 15) + 16 * qq) * 8 + j;
}

// prefill, step 1: grid (Tq, batch).  Rotates the keys of every position and writes keys and values into the cache.
template <typename CT, int D>
__global__ __launch_bounds__(256) void kv_write_kernel(AttnArgs a) {
    const int tq = blockIdx.x, b = blockIdx.y, t = threadIdx.x;
    const long row = (long)b * a.Tq + tq;
    const int pos = a.pos0 + tq;
    const int HD = a.H * D, GD = a.Hkv * D;
    CT* Kb = (CT*)a.kcache + (long)b * a.Hkv * a.max_len * D;
    CT* Vb = (CT*)a.vcache + (long)b * a.Hkv * a.max_len * D;
    for (int p = t; p < GD / 2; p += 256) {
        int kvh = p / (D / 2), i = p % (D / 2);
        int col = HD + kvh * D + 2 * i;
        float x0 = a.qkv[row * a.ldq + col] + a.bias[col], x1 = a.qkv[row * a.ldq + col + 1] + a.bias[col + 1], y0 = x0, y1 = x1;
        if (a.rope_cos) rope_pair(x0, x1, a.rope_cos[(long)pos * (D / 2) + i], a.rope_sin[(long)pos * (D / 2) + i], y0, y1);
        CT* Kh = Kb + (long)kvh * a.max_len * D;
        if (a.vt) { Kh[kfrag_index(pos, 2 * i, D)] = (CT)y0; Kh[kfrag_index(pos, 2 * i + 1, D)] = (CT)y1; }
        else { Kh[(long)pos * D + 2 * i] = (CT)y0; Kh[(long)pos * D + 2 * i + 1] = (CT)y1; }
    }
    for (int p = t; p < GD; p += 256) {
        int kvh = p / D, d = p % D;
        int col = HD + GD + p;
        const float val = a.qkv[row * a.ldq + col] + a.bias[col];
        if (a.vt) Vb[(long)kvh * a.max_len * D + vfrag_index(pos, d, D)] = (CT)val;
        else Vb[((long)kvh * a.max_len + pos) * D + d] = (CT)val;
    }
}

// prefill, step 1 for the fragment-major fp16 cache when the first position starts a 32-position chunk: one block per
// (chunk, KV head, batch row) writes the chunk's key and value fragments whole, 16 bytes per lane (the kernel above
// scatters two-byte elements from one small block per position).  Wavefront w: key fragment w (tile w / KD, kd w % KD)
// and value fragment w (dt = w).  grid (ceil(Tq / 32), Hkv, batch), D / 16 wavefronts.
template <int D>
__global__ __launch_bounds__(D * 4) void kv_write_frag_kernel(AttnArgs a) {
    constexpr int KD = D / 32;
    const int chunk = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int r = lane & 15, qq = lane >> 4;
    const int HD = a.H * D, GD = a.Hkv * D;
    const long cabs = (a.pos0 >> 5) + chunk;                     // chunk index in the cache (pos0 is a multiple of 32)
    half_t* Kh = (half_t*)a.kcache + ((long)b * a.Hkv + kvh) * a.max_len * D + cabs * (32 * D);
    half_t* Vh = (half_t*)a.vcache + ((long)b * a.Hkv + kvh) * (long)D * a.max_len + cabs * (32 * D);
    {   // keys: lane (r, qq) of fragment (tile, kd) holds position 8 (r / 4) + 4 tile + r % 4, d = 32 kd + 8 qq .. + 7
        const int tile = w / KD, kd = w % KD;
        const int tq = chunk * 32 + 8 * (r >> 2) + 4 * tile + (r & 3);
        const int d0 = 32 * kd + 8 * qq;
        half8 o = half8{0, 0, 0, 0, 0, 0, 0, 0};
        if (tq < a.Tq) {
            const long row = (long)b * a.Tq + tq;
            const int pos = a.pos0 + tq;
            const int col = HD + kvh * D + d0;
            const floatx4 x0 = *(const floatx4*)(a.qkv + row * a.ldq + col), x1 = *(const floatx4*)(a.qkv + row * a.ldq + col + 4);
            const floatx4 b0 = *(const floatx4*)(a.bias + col), b1 = *(const floatx4*)(a.bias + col + 4);
            float x[8];
#pragma unroll
            for (int j = 0; j < 4; ++j) { x[j] = x0[j] + b0[j]; x[4 + j] = x1[j] + b1[j]; }
#pragma unroll
            for (int pr = 0; pr < 4; ++pr) {
                float y0 = x[2 * pr], y1 = x[2 * pr + 1];
                if (a.rope_cos) {
                    const int i = d0 / 2 + pr;
                    rope_pair(x[2 * pr], x[2 * pr + 1], a.rope_cos[(long)pos * (D / 2) + i], a.rope_sin[(long)pos * (D / 2) + i], y0, y1);
                }
                o[2 * pr] = (half_t)y0; o[2 * pr + 1] = (half_t)y1;
            }
        }
        *(half8*)(Kh + (long)w * 512 + lane * 8) = o;
    }
    {   // values: lane (r, qq) of fragment dt holds d = 16 dt + r at positions 8 qq .. 8 qq + 7
        const int d = 16 * w + r;
        const int col = HD + GD + kvh * D + d;
        const float bv = a.bias[col];
        half8 o;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int tq = chunk * 32 + 8 * qq + j;
            o[j] = tq < a.Tq ? (half_t)(a.qkv[((long)b * a.Tq + tq) * a.ldq + col] + bv) : (half_t)0.0f;
        }
        *(half8*)(Vh + (long)w * 512 + lane * 8) = o;
    }
}

// prefill, step 2: grid (Tq, Hkv, batch).  Causal attention of query row tq over cache positions 0..pos0+tq.
// The reference adds -30000 to masked scores (TensorApplyCPU.cs:1016-1036, Decoder.cs:685-686); exp(-30000 - max)
// is exactly 0 in fp32, so leaving masked positions out gives the same sums.
template <typename CT, typename AT, int D, int G>
__global__ __launch_bounds__(256) void attn_prefill_kernel(AttnArgs a) {
    __shared__ AttnSmem<CT, D, G, 4> sm;
    const int tq = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z, t = threadIdx.x;
    const int kvc = a.kv_sub > 1 ? kvh / a.kv_sub : kvh;
    const long row = (long)b * a.Tq + tq;
    const int pos = a.pos0 + tq;
    for (int p = t; p < G * D / 2; p += 256) {
        int vec = p / (D / 2), i = p % (D / 2);
        int col = (kvh * G + vec) * D + 2 * i;
        float x0 = a.qkv[row * a.ldq + col] + a.bias[col], x1 = a.qkv[row * a.ldq + col + 1] + a.bias[col + 1], y0 = x0, y1 = x1;
        if (a.rope_cos) rope_pair(x0, x1, a.rope_cos[(long)pos * (D / 2) + i], a.rope_sin[(long)pos * (D / 2) + i], y0, y1);
        sm.q[vec * D + 2 * i] = a.scale * y0; sm.q[vec * D + 2 * i + 1] = a.scale * y1;
    }
    __syncthreads();
    const CT* Kb = (const CT*)a.kcache + ((long)b * a.Hkv + kvc) * a.max_len * D;
    const CT* Vb = (const CT*)a.vcache + ((long)b * a.Hkv + kvc) * a.max_len * D;
    const bool all_masked = a.lens && tq >= a.lens[b];          // (padded prompts start an empty cache: pos0 = 0)
    attn_core<CT, D, G, 4>(sm.q, Kb, Vb, all_masked ? a.pos0 + a.Tq : pos + 1, sm.m, sm.l, sm.acc, sm.out, all_masked);
    AT* out = (AT*)a.out + row * a.ld_out + kvh * G * D;
    for (int idx = t; idx < G * D; idx += 256) out[idx] = (AT)sm.out[idx];
}


// ------------------------------------------------------------------------------------------------
// MFMA attention (fp16 cache, head_dim 64 or 128), decode: one block per (batch row, KV head); the G query heads of
// the group use G of the 16 columns of v_mfma_f32_16x16x32_f16.  Keys and values are kept fragment-major (kfrag_index / vfrag_index), so every load is 1 KiB contiguous:
//   S[32 t][16 col]   = K tile (two 16-row A operands, rows permuted so that lane group q ends up with
//                       t = t0 + 8q .. 8q+7)  x  Q (B operand, kept in registers)
//   O^T[D][16 col]   += V^T tile (A operand: 16 d-rows x 32 t)  x  P (B operand: the lane's own 8 probabilities)
// Online softmax per column with one running maximum per wavefront; wavefronts take 32-row chunks round robin and
// are merged through LDS.  All arithmetic on scores, probabilities' sums and outputs is fp32.
// ------------------------------------------------------------------------------------------------
// SPLIT: a.S blocks (blockIdx.z) share one (batch row, KV head); chunks go round robin over all their wavefronts, every
// block leaves its unnormalised sums in an exchange area and the block that arrives last merges them in block order
// (same publication protocol as the split-K projections: agent-scope atomic stores, wait, counter; no spinning).
// For launches with fewer (row, head) pairs than CUs.
// The leading scalar arguments are everything the prologue's requests depend on: they are preloaded into scalar registers
// at wavefront start (see skinny_gemm_f16_kernel; at most 14 of them), so that no request waits for the argument struct.
// To fit, the pointers travel as one base (the key cache) and offsets from it in units of 256 bytes (every one of them is
// the start of a device allocation), and the small integers share words; attn_pack_args (host) builds them.  The struct's
// own copies of these fields are ignored.
struct AttnPacked {
    void* kcache; int d_vcache, d_qkv, d_pos, d_bias, d_ssq, d_rope_cos, d_rope_sin;   // offsets from kcache, 256-byte units
    int max_len; unsigned counts;     // H | Hkv << 8 | KS << 16 | (ssq ? 1 : 0) << 24 | (rope ? 1 : 0) << 25 | (ln ? 1 : 0) << 26
    int ldq, split_stride; unsigned ssq_dims;   // ssq_nt | ssq_ld << 16
};
template <int D, int G, bool SPLIT, bool SUB = false>      // SUB: groups of query heads share a KV head (AttnArgs::kv_sub > 1)
__global__ __launch_bounds__(D == 128 ? 256 : 512) void attn_mfma_kernel(void* kcache_, int d_vcache, int d_qkv, int d_pos, int d_bias, int d_ssq, int d_rope_cos,
                                                                       int d_rope_sin, int max_len_, unsigned counts, int ldq_, int split_stride_,
                                                                       unsigned ssq_dims, AttnArgs a) {
    {
        char* base = (char*)kcache_;
        auto at = [&](int d) { return (void*)(base + ((long)d << 8)); };
        a.kcache = kcache_; a.vcache = at(d_vcache); a.qkv = (const float*)at(d_qkv); a.d_pos = (const int*)at(d_pos); a.bias = (const float*)at(d_bias);
        a.ssq = (counts >> 24) & 1 ? (const float*)at(d_ssq) : nullptr; a.ln = (counts >> 26) & 1;
        a.rope_cos = (counts >> 25) & 1 ? (const float*)at(d_rope_cos) : nullptr; a.rope_sin = (counts >> 25) & 1 ? (const float*)at(d_rope_sin) : nullptr;
        a.max_len = max_len_; a.H = counts & 255; a.Hkv = (counts >> 8) & 255; a.KS = (counts >> 16) & 255; a.kv_sub = SUB ? counts >> 27 : 1;
        a.ldq = ldq_; a.split_stride = split_stride_; a.ssq_nt = ssq_dims & 0xffff; a.ssq_ld = ssq_dims >> 16;
    }
    constexpr int NW = D == 128 ? 4 : 8, NTH = NW * 64;
    constexpr int NCOL = G;                   // MFMA columns in use: the G query heads of the group
    constexpr int KD = D / 32, DT = D / 16;
    __shared__ float sIn[(G + 2) * D];
    __shared__ float sQ[16][D];
    __shared__ float sM[NW][16];
    __shared__ float sL[NW][16];
    __shared__ float sO[NW][D][16];
    const int t = threadIdx.x, lane = t & 63, w = __builtin_amdgcn_readfirstlane(t >> 6);
    // wavefront slot among all wavefronts of the pair, and their number
    const int gw = SPLIT ? (int)blockIdx.z * NW + w : w, GS = SPLIT ? a.S * NW : NW;
    const int r16 = lane & 15, q = lane >> 4;
    const int HD = a.H * D, GD = a.Hkv * D;
    // Groups of query heads that share a KV head (AttnArgs::kv_sub).  One block per pair: grid (Hkv, batch, kv_sub), so
    // that the cache addresses, which the first requests need, depend on blockIdx.x alone.  Several blocks per pair: grid
    // (Hkv * kv_sub, batch, blocks); kvh + 0.5 lies at least 1 / (2 kv_sub) from a multiple of kv_sub, far more than the
    // reciprocal's error.
    const int b = blockIdx.y;
    int kvh, kvc;
    if constexpr (!SUB) {
        kvh = kvc = blockIdx.x;
    } else if constexpr (SPLIT) {
        kvh = blockIdx.x;
        kvc = (int)(((float)kvh + 0.5f) * __builtin_amdgcn_rcpf((float)a.kv_sub));
    } else {
        kvc = blockIdx.x;
        kvh = kvc * a.kv_sub + (int)blockIdx.z;
    }
    // (the position is requested here and first used behind the prologue's other requests, which do not depend on it:
    // one memory round trip for both instead of one after the other)
    const int pos_base = *a.d_pos;
    half_t* Kb = (half_t*)a.kcache + ((long)b * a.Hkv + kvc) * a.max_len * D;
    half_t* Vt = (half_t*)a.vcache + ((long)b * a.Hkv + kvc) * (long)D * a.max_len;
    half8 kfA[2][KD], vfA[DT];
    auto load_chunk = [&](int c, half8 (&kf)[2][KD], half8 (&vf)[DT]) {
        const half_t* kc = Kb + (long)c * (32 * D) + lane * 8;
        const half_t* vc = Vt + (long)c * (32 * D) + lane * 8;
#pragma unroll
        for (int tile = 0; tile < 2; ++tile)
#pragma unroll
            for (int kd = 0; kd < KD; ++kd) kf[tile][kd] = load_once((const half8*)(kc + (tile * KD + kd) * 512));
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) vf[dt] = load_once((const half8*)(vc + dt * 512));
    };
    // Chunks of this wavefront: gw, gw + GS, ...  A CU accepts about 64 KiB of outstanding loads; a wavefront that
    // requests more stalls at the request, and loads that hit in L2 come back behind the misses queued before them.
    // So: the prologue's operands are requested first and the first chunk (8 KiB per wavefront, 64 KiB per CU) right
    // behind them; every later chunk is requested right before the chunk ahead of it is processed.  The first request
    // is unconditional so that the waits below are counted exactly; a first chunk that holds the row being appended
    // is requested again after the prologue.
    for (int i = t; i < 16 * D; i += NTH) (&sQ[0][0])[i] = 0.0f;
    int T, nchunks, n_own; bool validA;
    {
        constexpr int CPT = ((G + 2) * D + NTH - 1) / NTH;        // projection columns per thread
        constexpr int PPT = ((G + 1) * D / 2 + NTH - 1) / NTH;    // rotary pairs per thread
        // Every global load of the prologue is issued before the first use, and none of them waits for the argument
        // struct.  Order: the tile sums, the projection's partial sums and the bias (the first phase of the prologue needs
        // them; loads return in order), then the first chunk of keys and values, whose address does not depend on the
        // position, then the rotation of the position, which the second phase needs.
        // (the first four tile sums of a lane are requested without a wait of their own: a load-and-add loop would cost a
        // memory round trip ahead of every other request; they are added below in the same order)
        float ssq_part = 0.0f, ssq_v[4] = {0.0f, 0.0f, 0.0f, 0.0f}, ssum_v[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        if (a.ssq) {      // (unconditional requests at clamped indices; the values beyond the last tile are dropped below)
#pragma unroll
            for (int u = 0; u < 4; ++u) ssq_v[u] = a.ssq[(long)min(lane + 64 * u, a.ssq_nt - 1) * a.ssq_ld + b];
            if (a.ln) {
#pragma unroll
                for (int u = 0; u < 4; ++u) ssum_v[u] = a.ssq[(long)(a.ssq_nt + min(lane + 64 * u, a.ssq_nt - 1)) * a.ssq_ld + b];
            }
        }
        float part[CPT][8], bias[CPT], lnc[CPT];
        int pcol[CPT];
#pragma unroll
        for (int ci = 0; ci < CPT; ++ci) {
            const int idx = t + ci * NTH;
            pcol[ci] = 0;
#pragma unroll
            for (int k = 0; k < 8; ++k) part[ci][k] = 0.0f;
            if (idx < (G + 2) * D) {
                int col;
                if (idx < G * D) col = kvh * G * D + idx;
                else if (idx < (G + 1) * D) col = HD + kvc * D + (idx - G * D);
                else col = HD + GD + kvc * D + (idx - (G + 1) * D);
                pcol[ci] = col;
#pragma unroll
                for (int k = 0; k < 8; ++k) if (k < a.KS) part[ci][k] = a.qkv[k * a.split_stride + (long)b * a.ldq + col];
            }
            bias[ci] = a.bias[pcol[ci]];
            lnc[ci] = a.ln ? a.bias[a.ldq + pcol[ci]] : 0.0f;
        }
        __builtin_amdgcn_sched_barrier(0);
        load_chunk(min(gw, (int)(a.max_len >> 5) - 1), kfA, vfA);
        __builtin_amdgcn_sched_barrier(0);
        const int pos = pos_base;
        T = pos_base + 1; nchunks = (T + 31) / 32;
        n_own = nchunks > gw ? (nchunks - gw + GS - 1) / GS : 0;
        validA = gw < nchunks - 1;
        float rc[PPT], rs[PPT];
#pragma unroll
        for (int pi = 0; pi < PPT; ++pi) {
            const int p = t + pi * NTH;
            rc[pi] = 1.0f; rs[pi] = 0.0f;
            if (p < (G + 1) * D / 2 && a.rope_cos) { rc[pi] = a.rope_cos[(long)pos * (D / 2) + p % (D / 2)]; rs[pi] = a.rope_sin[(long)pos * (D / 2) + p % (D / 2)]; }
        }
        __builtin_amdgcn_sched_barrier(0);
        float rinv = 1.0f, mean = 0.0f;
        if (a.ssq) {
#pragma unroll
            for (int u = 0; u < 4; ++u) if (lane + 64 * u >= a.ssq_nt) ssq_v[u] = 0.0f;
            ssq_part = ((ssq_v[0] + ssq_v[1]) + ssq_v[2]) + ssq_v[3];
            for (int tt = lane + 256; tt < a.ssq_nt; tt += 64) ssq_part += a.ssq[(long)tt * a.ssq_ld + b];
            if (a.ln) {
#pragma unroll
                for (int u = 0; u < 4; ++u) if (lane + 64 * u >= a.ssq_nt) ssum_v[u] = 0.0f;
                float ssum_part = ((ssum_v[0] + ssum_v[1]) + ssum_v[2]) + ssum_v[3];
                for (int tt = lane + 256; tt < a.ssq_nt; tt += 64) ssum_part += a.ssq[(long)(a.ssq_nt + tt) * a.ssq_ld + b];
                mean = wave_sum(ssum_part) * a.inv_h;
                rinv = 1.0f / sqrtf(fmaxf(wave_sum(ssq_part) * a.inv_h - mean * mean, 0.0f) + a.eps);
            } else {
                rinv = 1.0f / sqrtf(wave_sum(ssq_part) * a.inv_h + a.eps);
            }
        }
#pragma unroll
        for (int ci = 0; ci < CPT; ++ci) {
            const int idx = t + ci * NTH;
            if (idx < (G + 2) * D) {
                float s = part[ci][0];
#pragma unroll
                for (int k = 1; k < 8; ++k) if (k < a.KS) s += part[ci][k];
                for (int k = 8; k < a.KS; ++k) s += a.qkv[k * a.split_stride + (long)b * a.ldq + pcol[ci]];     // (more than eight splits: wide models at batches above 64)
                sIn[idx] = (s - mean * lnc[ci]) * rinv + bias[ci];      // (LayerNorm: the mean's share of the product; 0 otherwise)
            }
        }
        __syncthreads();
#pragma unroll
        for (int pi = 0; pi < PPT; ++pi) {
            const int p = t + pi * NTH;
            if (p < (G + 1) * D / 2) {
                const int vec = p / (D / 2), i = p % (D / 2);
                float x0 = sIn[vec * D + 2 * i], x1 = sIn[vec * D + 2 * i + 1], y0 = x0, y1 = x1;
                if (a.rope_cos) rope_pair(x0, x1, rc[pi], rs[pi], y0, y1);
                // (scores are kept in units of log 2, so that the exponentials below are bare v_exp_f32)
                if (vec < G) { sQ[vec][2 * i] = (a.scale * 1.44269504f) * y0; sQ[vec][2 * i + 1] = (a.scale * 1.44269504f) * y1; }
                else { Kb[kfrag_index(pos, 2 * i, D)] = (half_t)y0; Kb[kfrag_index(pos, 2 * i + 1, D)] = (half_t)y1; }
            }
        }
        for (int d = t; d < D; d += NTH) Vt[vfrag_index(pos, d, D)] = (half_t)sIn[(G + 1) * D + d];
        __threadfence_block();
    }
    __syncthreads();

    // B operand of the score product: lane (col = r16, q) holds Q[col][kd*32 + 8q .. +7]
    half8 qf[KD];
#pragma unroll
    for (int kd = 0; kd < KD; ++kd)
#pragma unroll
        for (int j = 0; j < 8; ++j) qf[kd][j] = r16 < NCOL ? (half_t)sQ[r16][kd * 32 + 8 * q + j] : (half_t)0.0f;      // columns beyond the group: zero queries, scores 0
    // last position the columns may attend to (the same for all: one query position per sequence)
    const int tmax = T - 1;

    float m_run = -INFINITY, l_run = 0.0f;
    floatx4 acc_o[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) acc_o[dt] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};

    auto do_chunk = [&](int c, half8 (&kf)[2][KD], half8 (&vf)[DT]) {
        const int t0 = c * 32;
        floatx4 sA = floatx4{0.0f, 0.0f, 0.0f, 0.0f}, sB = sA;
#pragma unroll
        for (int kd = 0; kd < KD; ++kd) {
            sA = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf[0][kd], qf[kd], sA, 0, 0, 0);
            sB = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf[1][kd], qf[kd], sB, 0, 0, 0);
        }
        // this lane: column r16, positions t0 + 8q + j  (j < 4 from sA, j >= 4 from sB)
        float s[8];
#pragma unroll
        for (int j = 0; j < 4; ++j) { s[j] = sA[j]; s[4 + j] = sB[j]; }
        if (t0 + 31 > tmax) {          // only the chunk that holds the newest position has positions to hide
#pragma unroll
            for (int j = 0; j < 8; ++j) if (t0 + 8 * q + j > tmax) s[j] = -INFINITY;
        }
        float cm = -INFINITY;
#pragma unroll
        for (int j = 0; j < 8; ++j) cm = fmaxf(cm, s[j]);
        cm = max_xor32(max_xor16(cm));
        // (a chunk that is processed has a visible position, so m_new is finite; exp2(-inf) = 0 covers hidden positions
        // and the first chunk's m_run)
        const float m_new = fmaxf(m_run, cm);
        const float corr = __builtin_amdgcn_exp2f(m_run - m_new);
        half8 pf;
        float psum = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float p = __builtin_amdgcn_exp2f(s[j] - m_new);
            psum += p;
            pf[j] = (half_t)p;
        }
        l_run = l_run * corr + psum;
        m_run = m_new;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
            for (int i = 0; i < 4; ++i) acc_o[dt][i] *= corr;
            acc_o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vf[dt], pf, acc_o[dt], 0, 0, 0);
        }
    };
    // Register sets are never carried around a loop (the copies at the back edge would wait for loads in flight) and a
    // request never sits under a condition of its own (every later wait would have to cover it).  The first NFX chunks
    // form a chain of stages: a stage either requests the next chunk and processes its own, or processes the last
    // one; longer contexts continue in groups of NL chunks requested together.
    if (n_own >= 1 && !validA) load_chunk(gw, kfA, vfA);
    constexpr int NFX = D == 128 ? 3 : 7, NL = D == 128 ? 2 : 4;
    auto group = [&](auto nc, int c0) {
        constexpr int N = decltype(nc)::value;
        half8 kr[N][2][KD], vr[N][DT];
#pragma unroll
        for (int g = 0; g < N; ++g) load_chunk(c0 + g * GS, kr[g], vr[g]);
#pragma unroll
        for (int g = 0; g < N; ++g) do_chunk(c0 + g * GS, kr[g], vr[g]);
    };
    auto chain = [&](auto self, auto gc, half8 (&kc)[2][KD], half8 (&vc)[DT]) -> void {
        constexpr int g = decltype(gc)::value;           // kc, vc: chunk gw + g GS, requested
        const int cg = gw + g * GS;
        if constexpr (g == NFX) {
            do_chunk(cg, kc, vc);
            int c = cg + GS;
            for (; c + (NL - 1) * GS < nchunks; c += NL * GS) group(std::integral_constant<int, NL>{}, c);
            if constexpr (NL == 4) {
                if (c + 2 * GS < nchunks) group(std::integral_constant<int, 3>{}, c);
                else if (c + GS < nchunks) group(std::integral_constant<int, 2>{}, c);
                else if (c < nchunks) group(std::integral_constant<int, 1>{}, c);
            } else {
                if (c < nchunks) group(std::integral_constant<int, 1>{}, c);
            }
        } else {
            if (cg + GS < nchunks) {
                half8 kn[2][KD], vn[DT];
                load_chunk(cg + GS, kn, vn);
                do_chunk(cg, kc, vc);
                self(self, std::integral_constant<int, g + 1>{}, kn, vn);
            } else {
                do_chunk(cg, kc, vc);
            }
        }
    };
    if (n_own >= 1) chain(chain, std::integral_constant<int, 0>{}, kfA, vfA);
    // the four lane groups of a column saw different positions: add their sums (the maximum is already common)
    l_run = sum_xor32(sum_xor16(l_run));
    if (q == 0) { sM[w][r16] = m_run; sL[w][r16] = l_run; }
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int i = 0; i < 4; ++i) sO[w][dt * 16 + 4 * q + i][r16] = acc_o[dt][i];
    __syncthreads();
    if constexpr (SPLIT) {
        // block sums relative to the block maximum -> exchange area [pair][block][NCOL D + 2 NCOL] floats
        __shared__ int s_last;
        const int pair = b * (int)gridDim.x + kvh;
        const long per = (long)NCOL * D + 2 * NCOL;
        float* mine = a.xchg + ((long)pair * a.S + blockIdx.z) * per;
        for (int idx = t; idx < NCOL * D; idx += NTH) {
            const int col = idx % NCOL, d = idx / NCOL;
            float M = -INFINITY;
#pragma unroll
            for (int i = 0; i < NW; ++i) M = fmaxf(M, sM[i][col]);
            float L = 0.0f, O = 0.0f;
#pragma unroll
            for (int i = 0; i < NW; ++i) {
                const float wgt = (sM[i][col] == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f(sM[i][col] - M);
                L += sL[i][col] * wgt;
                O += sO[i][d][col] * wgt;
            }
            __hip_atomic_store(mine + idx, O, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (d == 0) {
                __hip_atomic_store(mine + NCOL * D + col, M, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(mine + NCOL * D + NCOL + col, L, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        // (same publication protocol as the split-K projections' exchange, whose comment lists the instruction sequence it
        // rests on: write-through atomic stores, vmcnt(0), block barrier, atomic add, atomic loads in the last arriver)
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");            // the stores have reached the point of coherence
        __syncthreads();
        if (t == 0) s_last = __hip_atomic_fetch_add(a.xcount + pair, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == a.S - 1;
        __syncthreads();
        if (!s_last) return;
        // every block of the pair has published (its count came after its stores): merge in block order
        const float* base = a.xchg + (long)pair * a.S * per;
        for (int idx = t; idx < NCOL * D; idx += NTH) {
            const int col = idx % NCOL, d = idx / NCOL;
            float M = -INFINITY;
            for (int s = 0; s < a.S; ++s) M = fmaxf(M, __hip_atomic_load(base + s * per + NCOL * D + col, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
            float L = 0.0f, O = 0.0f;
            for (int s = 0; s < a.S; ++s) {
                const float ms = __hip_atomic_load(base + s * per + NCOL * D + col, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                const float wgt = (ms == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f(ms - M);
                L += __hip_atomic_load(base + s * per + NCOL * D + NCOL + col, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) * wgt;
                O += __hip_atomic_load(base + s * per + idx, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) * wgt;
            }
            const float o = O / L;
            const int kcol = (kvh * G + col) * D + d;
            if (a.out_kt > 0) ((half_t*)a.out)[xpack_index(b, kcol, a.out_kt)] = (half_t)o;
            else ((half_t*)a.out)[(long)b * a.ld_out + kcol] = (half_t)o;
        }
        if (t == 0) __hip_atomic_store(a.xcount + pair, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);       // ready for the next launch
        return;
    }
    for (int idx = t; idx < NCOL * D; idx += NTH) {
        const int col = idx % NCOL, d = idx / NCOL;
        float M = -INFINITY;
#pragma unroll
        for (int i = 0; i < NW; ++i) M = fmaxf(M, sM[i][col]);
        float L = 0.0f, O = 0.0f;
#pragma unroll
        for (int i = 0; i < NW; ++i) {
            const float wgt = (sM[i][col] == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f(sM[i][col] - M);
            L += sL[i][col] * wgt;
            O += sO[i][d][col] * wgt;
        }
        const float o = O / L;
        const int g = col;
        const int kcol = (kvh * G + g) * D + d;
        if (a.out_kt > 0) ((half_t*)a.out)[xpack_index(b, kcol, a.out_kt)] = (half_t)o;
        else ((half_t*)a.out)[(long)b * a.ld_out + kcol] = (half_t)o;
    }
}

// Prefill variant: a wavefront owns QB = 16 / G consecutive query positions (the 16 MFMA columns are its positions x
// the G query heads of the group), so there is no merge across wavefronts.  The NW wavefronts of a block sit at
// neighbouring positions and need the same chunks: the block fetches every 32-position chunk of its causal prefix once,
// straight into LDS (four stages, requested two chunks ahead; wavefront w brings fragments w, w + NW, ...), and all
// wavefronts read their MFMA operands from there.  (With every wavefront streaming its own prefix the kernel was bound
// by L2: the L1 holds two chunks and the wavefronts drift apart.)  grid (ceil(Tq / (QB NW)), Hkv, batch).
// RAGGED: sequences padded to one length (a.lens).  A query row at or beyond its sequence's length attends to every
// column of the padded sequence with scores rounded as the float32 addition of -30000 rounds them; every chunk then
// takes the masked path and a block that holds such a row walks all chunks.
// NQ: groups of 16 MFMA columns per wavefront (NQ QB consecutive positions): every key and value fragment read from
// LDS then serves NQ MFMAs.
template <int D, int G, bool RAGGED = false, int NQ = 1>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(D == 64 ? (NQ == 1 && !RAGGED ? 6 : 4) : 2))) void attn_mfma_prefill_kernel(AttnArgs a) {
    constexpr int NW = 8;
    constexpr int QB = 16 / G, KD = D / 32, DT = D / 16;
    constexpr int NF = 2 * KD + DT;          // 1 KiB fragments per chunk: keys (tile, kd), then values (dt)
    constexpr int FPW = NF / NW;             // fragments a wavefront brings per chunk
    static_assert(NF % NW == 0, "fragments must divide among the wavefronts");
    // LDS layout, as one struct so that the compiler lays the regions out and the assertions below are about what it did.
    // The invariant they state: a direct-to-LDS request may land at any time between its issue and the wait at the barrier
    // two chunks later, so the bytes it targets (one stage) must belong to nothing that any wavefront reads or writes in
    // that window: the stages are an array of their own, apart from the per-wavefront staging of queries and outputs (which
    // is written right behind barriers), and a request issued at barrier j targets the stage of chunk j + AHEAD, while
    // the wavefronts between barriers j and j + 1 read the stages of chunks j (values) and j + 1 (keys) and older
    // requests are still landing in the stage of chunk j + 1.
    constexpr int STAGES = 4, AHEAD = 2;
    struct PrefillLds {
        // per wavefront: the queries [16 columns][D] as fp16, later the outputs [D / 2][16 columns] as fp32, half of them
        // at a time (2 KiB at head size 64: with the stages 48.5 KiB per block, three blocks per compute unit)
        __attribute__((aligned(16))) half_t sbuf[NW][D * 16];
        float sl[NW][16];
        // the chunk stages, of their own: with two of them in the query / output staging area (16 KiB less, a third block
        // per compute unit at head size 64) single rows of the wavefronts that own that area came out wrong now and then
        __attribute__((aligned(16))) half_t sstage[STAGES][NF * 512];
    };
    static_assert((STAGES & (STAGES - 1)) == 0, "stage_of() masks the chunk number");
    static_assert(AHEAD + 2 <= STAGES, "the stage a request lands in (chunk j + AHEAD) must differ from the stages read between barriers j and j + 1 "
                                       "(chunks j, j + 1) and from the one the wavefronts that have not yet passed barrier j still read (chunk j - 1)");
    static_assert(sizeof(float) * (D / 2) * 16 <= sizeof(half_t) * D * 16, "half of a wavefront's outputs [D / 2][16] as fp32 must fit its query staging slice");
    static_assert(offsetof(PrefillLds, sstage) >= offsetof(PrefillLds, sl) + sizeof(float) * NW * 16 &&
                  offsetof(PrefillLds, sl) >= offsetof(PrefillLds, sbuf) + sizeof(half_t) * NW * D * 16, "staging, sums and stages do not overlap");
    static_assert(offsetof(PrefillLds, sstage) % 16 == 0 && (NF * 1024) % 16 == 0, "16-byte fragment reads and direct-to-LDS writes are aligned");
    static_assert((NF - 1) * 1024 + 63 * 16 + 16 <= NF * 1024, "the last fragment read of a stage (offset (NF - 1) KiB, lane 63) ends inside the stage");
    static_assert(FPW * NW == NF, "the wavefronts' requests cover a stage exactly: fragments w, w + NW, ...");
    // blocks per compute unit the launch bounds ask for (waves per SIMD x 4 SIMDs / 8 wavefronts per block): their LDS must fit
    constexpr int BLOCKS_PER_CU = (D == 64 ? (NQ == 1 && !RAGGED ? 6 : 4) : 2) * 4 / NW;
    static_assert(sizeof(PrefillLds) * BLOCKS_PER_CU <= 160 * 1024, "the resident blocks' LDS fits the 160 KiB of a compute unit");
    // (the struct above is the layout the assertions are about; the regions themselves are three objects of the same
    // shapes, which the compiler keeps apart by construction: allocated as one object, the register allocator of this
    // 80-register build put a spill reload into the chunk loops)
    __shared__ __attribute__((aligned(16))) half_t sbuf[NW][D * 16];
    __shared__ float sl[NW][16];
    __shared__ __attribute__((aligned(16))) half_t sstage[STAGES * NF * 512];
    static_assert(sizeof(sbuf) == sizeof(PrefillLds::sbuf) && sizeof(sl) == sizeof(PrefillLds::sl) && sizeof(sstage) == sizeof(PrefillLds::sstage),
                  "the allocated regions have the asserted shapes");
    const int lane = threadIdx.x & 63, w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r16 = lane & 15, q = lane >> 4;
    const int kvh = blockIdx.y, b = blockIdx.z;
    const int kvc = a.kv_sub > 1 ? kvh / a.kv_sub : kvh;       // (groups of query heads that share a KV head, see AttnArgs::kv_sub)
    const int tq0 = (blockIdx.x * NW + w) * (QB * NQ);
    const bool active = tq0 < a.Tq;          // wavefronts beyond the prompt still fetch their share of every chunk
    const int pos_base = a.pos0 + tq0, T = min(pos_base + QB * NQ, a.pos0 + a.Tq);
    // chunks of the block: up to the last position of its last active wavefront
    const int tq_last = min(a.Tq, (int)(blockIdx.x + 1) * NW * QB * NQ);
    const int len_b = RAGGED ? a.lens[b] : 0x7fffffff;
    const int Ttot = a.pos0 + a.Tq;
    const int nchunks = (RAGGED && tq_last > len_b) ? (Ttot + 31) / 32 : (a.pos0 + tq_last + 31) / 32;
    const half_t* Kb = (const half_t*)a.kcache + ((long)b * a.Hkv + kvc) * a.max_len * D;
    const half_t* Vt = (const half_t*)a.vcache + ((long)b * a.Hkv + kvc) * (long)D * a.max_len;
    typedef const void __attribute__((address_space(1)))* gptr_t;
    typedef void __attribute__((address_space(3)))* lptr_t;
    auto stage_of = [&](int c) -> half_t* { return sstage + (c & (STAGES - 1)) * (NF * 512); };
    auto fetch_to = [&](int c, int slot) {   // this wavefront's fragments of chunk c -> the stage of chunk `slot`
        half_t* dst = stage_of(slot);
#pragma unroll
        for (int i = 0; i < FPW; ++i) {
            const int f = w + i * NW;
            const half_t* src = (f < 2 * KD ? Kb + (long)c * (32 * D) + f * 512 : Vt + (long)c * (32 * D) + (f - 2 * KD) * 512) + lane * 8;
            __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)(dst + f * 512), 16, 0, 0);
        }
    };
    static_assert(AHEAD == 2, "the two requests below are the AHEAD chunks in flight before barrier 0");
    fetch_to(0, 0);
    fetch_to(min(1, nchunks - 1), 1);

    // queries: projection + bias, rotary embedding, 1 / sqrt(d); columns beyond the prompt stay zero.  A lane takes
    // four consecutive elements (two rotary pairs) of a column at a time; the requests of four such pieces go out
    // together (one memory round trip per batch: piece by piece the block spent longer here than in its chunks)
    half_t* sq = sbuf[w];
    half8 qf[NQ][KD];
#pragma unroll
    for (int g2 = 0; g2 < NQ; ++g2) {
        constexpr int PIECES = 16 * D / 4 / 64, BATCH = 4;       // pieces per lane, pieces requested together
        static_assert(PIECES % BATCH == 0, "whole batches");
        const float qs = a.scale * 1.44269504f;                  // (scores are kept in units of log 2, so that the exponentials below are bare v_exp_f32)
#pragma unroll
        for (int b0 = 0; b0 < PIECES; b0 += BATCH) {
            floatx4 xv[BATCH], bv[BATCH]; floatx2 cv[BATCH], sv[BATCH]; bool ok[BATCH];
#pragma unroll
            for (int u = 0; u < BATCH; ++u) {
                const int p = lane + 64 * (b0 + u);
                const int col = p / (D / 4), i4 = p % (D / 4);
                const int qi = col / G, g = col % G;
                ok[u] = active && qi < QB && tq0 + g2 * QB + qi < a.Tq;      // (G that does not divide 16: the last 16 - QB G columns stay empty)
                const int qic = ok[u] ? g2 * QB + qi : 0;        // (a valid address either way; the value is dropped)
                const long row = (long)b * a.Tq + min(tq0, a.Tq - 1) + qic;
                const int c0 = (kvh * G + g) * D + 4 * i4;
                xv[u] = *(const floatx4*)(a.qkv + row * a.ldq + c0);
                bv[u] = *(const floatx4*)(a.bias + c0);
                if (a.rope_cos) {
                    const long ro = (long)(min(pos_base, a.pos0 + a.Tq - 1) + qic) * (D / 2) + 2 * i4;
                    cv[u] = *(const floatx2*)(a.rope_cos + ro); sv[u] = *(const floatx2*)(a.rope_sin + ro);
                }
            }
#pragma unroll
            for (int u = 0; u < BATCH; ++u) {
                const int p = lane + 64 * (b0 + u);
                const int col = p / (D / 4), i4 = p % (D / 4);
                floatx4 y;
#pragma unroll
                for (int pr = 0; pr < 2; ++pr) {
                    const float x0 = xv[u][2 * pr] + bv[u][2 * pr], x1 = xv[u][2 * pr + 1] + bv[u][2 * pr + 1];
                    float y0 = x0, y1 = x1;
                    if (a.rope_cos) rope_pair(x0, x1, cv[u][pr], sv[u][pr], y0, y1);
                    y[2 * pr] = ok[u] ? qs * y0 : 0.0f; y[2 * pr + 1] = ok[u] ? qs * y1 : 0.0f;
                }
                half4 yh;
#pragma unroll
                for (int e4 = 0; e4 < 4; ++e4) yh[e4] = (half_t)y[e4];
                *(half4*)(sq + col * D + 4 * i4) = yh;
            }
        }
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int kd = 0; kd < KD; ++kd)
#pragma unroll
            for (int j = 0; j < 8; ++j) qf[g2][kd][j] = sq[r16 * D + kd * 32 + 8 * q + j];
        __builtin_amdgcn_wave_barrier();
    }
    bool fully[NQ]; int tmax[NQ];
    float l_run[NQ];
    floatx4 acc_o[NQ][DT];
#pragma unroll
    for (int g2 = 0; g2 < NQ; ++g2) {
        fully[g2] = RAGGED && tq0 + g2 * QB + r16 / G >= len_b;              // this lane's query row has every column masked
        tmax[g2] = fully[g2] ? Ttot - 1 : pos_base + g2 * QB + r16 / G;      // last position this lane's column may attend to
        l_run[g2] = 0.0f;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) acc_o[g2][dt] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    }
    // Chunks [0, n_full) lie entirely at or below this wavefront's first query position; chunks from n_own on lie
    // entirely behind its last one (the block's later wavefronts still need them).
    const std::integral_constant<bool, false> plain; const std::integral_constant<bool, true> masked;
    const bool wave_fully = RAGGED && active && min(tq0 + QB * NQ, a.Tq) > len_b;      // its last query row lies beyond the sequence's length
    const int n_own = active ? (wave_fully ? (Ttot + 31) / 32 : (T + 31) / 32) : 0;
    const int n_full = RAGGED ? 0 : min(n_own, (pos_base + 1) / 32);
    // The walk over the chunks.  An iteration holds the scores of its chunk (their MFMAs were issued in the iteration
    // before).  It requests the key fragments of the next chunk and the value fragments of its own from LDS, runs the
    // exponentials of its scores, issues the next chunk's score MFMAs and, last, its own value MFMAs: the matrix pipe
    // and the LDS reads work under the per-score arithmetic instead of in turns with it.
    // Barrier j (one per chunk, and one more): chunk j has landed for everybody and nobody reads chunk j - 2 any
    // more, whose stage the request for chunk j + 2 then overwrites.  No branches: behind the last chunk the last
    // chunk is requested again, into a stage nobody reads any more, so that the count of outstanding requests is the
    // same at every barrier.  Every wavefront passes barriers 0 ... nchunks whatever its own number of chunks.
    // The fragment reads and their waits are written out: the compiler cannot tell which LDS bytes a request in
    // flight will write and would wait for all of them before any LDS read.
    auto wait_barrier = [&](int j) {
        asm volatile("s_waitcnt vmcnt(%0)" :: "n"(FPW) : "memory");
        __builtin_amdgcn_s_barrier();
        fetch_to(min(j + AHEAD, nchunks - 1), j + AHEAD);
    };
    {
        half8 kf[2][KD], vf[DT];
        floatx4 sA[NQ], sB[NQ];
        // (hand-written reads: the compiler takes their results as present once issued.  Every read_k is tied by k_landed /
        // k_landed_alone and every read_v by v_landed, in the basic block that issues it, before anything uses or reuses
        // the registers; tests/test_asm_hazards.py scans the generated code for a read without such a wait.)
        auto read_k = [&](int c) {
            const unsigned sa = (unsigned)(size_t)(lptr_t)stage_of(c) + lane * 16;
#pragma unroll
            for (int tile = 0; tile < 2; ++tile)
#pragma unroll
                for (int kd = 0; kd < KD; ++kd) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=&v"(kf[tile][kd]) : "v"(sa), "n"((tile * KD + kd) * 1024) : "memory");
        };
        auto read_v = [&](int c, half8 (&vf)[DT]) {
            const unsigned sa = (unsigned)(size_t)(lptr_t)stage_of(c) + lane * 16;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=&v"(vf[dt]) : "v"(sa), "n"((2 * KD + dt) * 1024) : "memory");
        };
        // The key fragments have arrived once only the reads issued behind them are outstanding.  (A count that lets
        // a read land late hands its registers to the compiler while the LDS still writes them: an address kept there
        // is then overwritten.)
        auto k_landed = [&]() {              // in a chunk's iteration: the DT value reads follow the key reads
            if constexpr (KD == 2)
                asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(kf[0][0]), "+v"(kf[0][1]), "+v"(kf[1][0]), "+v"(kf[1][1]) : "n"(DT) : "memory");
            else
                asm volatile("s_waitcnt lgkmcnt(%8)" : "+v"(kf[0][0]), "+v"(kf[0][1]), "+v"(kf[0][2]), "+v"(kf[0][3]), "+v"(kf[1][0]), "+v"(kf[1][1]), "+v"(kf[1][2]), "+v"(kf[1][3]) : "n"(DT) : "memory");
        };
        auto k_landed_alone = [&]() {        // before the first chunk: nothing follows the key reads
            if constexpr (KD == 2)
                asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(kf[0][0]), "+v"(kf[0][1]), "+v"(kf[1][0]), "+v"(kf[1][1]) :: "memory");
            else
                asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(kf[0][0]), "+v"(kf[0][1]), "+v"(kf[0][2]), "+v"(kf[0][3]), "+v"(kf[1][0]), "+v"(kf[1][1]), "+v"(kf[1][2]), "+v"(kf[1][3]) :: "memory");
        };
        auto v_landed = [&](half8 (&vf)[DT]) {
            if constexpr (D == 64)
                asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(vf[0]), "+v"(vf[1]), "+v"(vf[2]), "+v"(vf[3]) :: "memory");
            else
                asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(vf[0]), "+v"(vf[1]), "+v"(vf[2]), "+v"(vf[3]), "+v"(vf[4]), "+v"(vf[5]), "+v"(vf[6]), "+v"(vf[7]) :: "memory");
        };
        // Scores are kept relative to a reference m_ref per column (units of log 2): the score MFMAs start from
        // -m_ref, so that their outputs are s - m_ref and the probabilities are bare exponentials of them.  The
        // reference is the column's running maximum as of the last time it was moved; it is moved (and the running
        // outputs and sums rescaled) only in a chunk where some score exceeds it by more than SLACK: probabilities
        // then lie in (0, 2^SLACK], well inside fp16 and fp32 range, and the quotient of output and sum does not
        // depend on the reference.  Most chunks therefore take neither the cross-lane maximum nor the 4 DT
        // multiplications of the running outputs.
        constexpr float SLACK = 8.0f;
        float m_ref[NQ];
        floatx4 nmq[NQ];                                     // -m_ref four times: the score MFMAs' starting accumulator
#pragma unroll
        for (int g2 = 0; g2 < NQ; ++g2) { m_ref[g2] = 0.0f; nmq[g2] = floatx4{0.0f, 0.0f, 0.0f, 0.0f}; sA[g2] = nmq[g2]; sB[g2] = nmq[g2]; }
        auto scores = [&]() {
#pragma unroll
            for (int kd = 0; kd < KD; ++kd)
#pragma unroll
                for (int g2 = 0; g2 < NQ; ++g2) {
                    sA[g2] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf[0][kd], qf[g2][kd], kd == 0 ? nmq[g2] : sA[g2], 0, 0, 0);
                    sB[g2] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf[1][kd], qf[g2][kd], kd == 0 ? nmq[g2] : sB[g2], 0, 0, 0);
                }
        };
        // A row beyond its sequence's length: round the new scores (units of log 2) as s + (-30000) rounds them in
        // natural units.  (A per-lane branch: it sits where no LDS read is in flight.)
        auto round_scores = [&]() {
#pragma unroll
            for (int g2 = 0; g2 < NQ; ++g2)
                if (RAGGED && fully[g2]) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const float an = (sA[g2][j] + m_ref[g2]) * 0.69314718f + (-30000.0f), bn = (sB[g2][j] + m_ref[g2]) * 0.69314718f + (-30000.0f);
                        sA[g2][j] = (an - (-30000.0f)) * 1.44269504f - m_ref[g2]; sB[g2][j] = (bn - (-30000.0f)) * 1.44269504f - m_ref[g2];
                    }
                }
        };
        auto mask_scores = [&](int c) {
            const int t0 = c * 32;
#pragma unroll
            for (int g2 = 0; g2 < NQ; ++g2)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if (t0 + 8 * q + j > tmax[g2]) sA[g2][j] = -INFINITY;
                    if (t0 + 8 * q + 4 + j > tmax[g2]) sB[g2][j] = -INFINITY;
                }
        };
        auto local_max = [&](int g2) {
            float lm = sA[g2][0];
#pragma unroll
            for (int j = 1; j < 8; ++j) lm = fmaxf(lm, j < 4 ? sA[g2][j] : sB[g2][j - 4]);
            return lm;
        };
        // Moves the reference of every column to its maximum in the chunk at hand where that is larger, and rescales
        // what has been accumulated.  Inside the loop this is a rarely taken branch, and the updates are written as
        // instructions on the registers in place: left to the compiler, the join behind the branch costs a copy of
        // every running output in every chunk.  The compiler inserts no wait states between an MFMA and an
        // instruction it cannot see, so the idle instructions in front (tied to the outputs, hence behind the MFMAs
        // that produce them) provide the distance the hardware requires between the two.
        auto move_reference = [&]() {
#pragma unroll
            for (int g2 = 0; g2 < NQ; ++g2) {
                const float cm = max_xor32(max_xor16(local_max(g2)));
                float d = fmaxf(cm, 0.0f);
                float corr = __builtin_amdgcn_exp2f(-d);
                // (tied to the factor as well: an exponential's result also needs a distance the compiler only keeps
                // for instructions it can see)
                if constexpr (DT == 4)
                    asm volatile("s_nop 15\n\ts_nop 15" : "+v"(d), "+v"(corr), "+v"(acc_o[g2][0]), "+v"(acc_o[g2][1]), "+v"(acc_o[g2][2]), "+v"(acc_o[g2][3]));
                else
                    asm volatile("s_nop 15\n\ts_nop 15" : "+v"(d), "+v"(corr), "+v"(acc_o[g2][0]), "+v"(acc_o[g2][1]), "+v"(acc_o[g2][2]), "+v"(acc_o[g2][3]), "+v"(acc_o[g2][4]), "+v"(acc_o[g2][5]), "+v"(acc_o[g2][6]), "+v"(acc_o[g2][7]));
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) asm volatile("v_mul_f32 %0, %0, %1" : "+v"(acc_o[g2][dt][i]) : "v"(corr));
                asm volatile("v_mul_f32 %0, %0, %1" : "+v"(l_run[g2]) : "v"(corr));
                if (RAGGED) asm volatile("v_add_f32 %0, %0, %1" : "+v"(m_ref[g2]) : "v"(d));       // (only the rounding of rows beyond their length reads it)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    asm volatile("v_sub_f32 %0, %0, %1" : "+v"(sA[g2][j]) : "v"(d));
                    asm volatile("v_sub_f32 %0, %0, %1" : "+v"(sB[g2][j]) : "v"(d));
                    asm volatile("v_sub_f32 %0, %0, %1" : "+v"(nmq[g2][j]) : "v"(d));
                }
            }
        };
        // One chunk.  Its value MFMAs are issued last and run under the next chunk's comparisons and its wait at the
        // barrier.  They are written as instructions that accumulate in place: the register allocator otherwise
        // writes results over dead fragments and copies them back, one copy per running output per chunk.  Nothing
        // reads the running outputs before the same place one chunk later except the rescaling and the epilogue,
        // which keep their own distance; the idle instruction in front covers the probabilities just converted.
        auto iter = [&](auto masked_c, int c) {
            constexpr bool MASKED = decltype(masked_c)::value;
            if (MASKED) mask_scores(c);
            {   // any score more than SLACK above its column's reference?  (no LDS read is in flight here)
                float lm = local_max(0);
#pragma unroll
                for (int g2 = 1; g2 < NQ; ++g2) lm = fmaxf(lm, local_max(g2));
                if (__builtin_amdgcn_ballot_w64(lm > SLACK) != 0) move_reference();
            }
            wait_barrier(c + 1);
            read_k(c + 1);                   // (behind the wavefront's last chunk: any stage, the scores are not used)
            read_v(c, vf);
            half8 pf[NQ];
#pragma unroll
            for (int g2 = 0; g2 < NQ; ++g2) {
                float psum = 0.0f;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const float p = __builtin_amdgcn_exp2f(j < 4 ? sA[g2][j] : sB[g2][j - 4]);
                    psum += p;
                    pf[g2][j] = (half_t)p;
                }
                l_run[g2] += psum;
            }
            k_landed();
            scores();                        // (the next chunk's scores, into the registers the exponentials have just read)
            // The value fragments are tied in the basic block that requested them, behind everything above (by now
            // they have long arrived).  Tied across a branch, the compiler may copy the registers on the edge, before
            // the wait: a copy of a register whose read is still in flight.
            __builtin_amdgcn_sched_barrier(0);
            v_landed(vf);
            if constexpr (NQ == 1) asm volatile("s_nop 4" : "+v"(pf[0]));
            else asm volatile("s_nop 4" : "+v"(pf[0]), "+v"(pf[NQ - 1]));
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int g2 = 0; g2 < NQ; ++g2)
                    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(acc_o[g2][dt]) : "v"(vf[dt]), "v"(pf[g2]));
            round_scores();
        };
        // barrier 0, the first chunk's scores and every column's first reference
        wait_barrier(0);
        if (n_own > 0) {
            read_k(0);
            k_landed_alone();
            scores();
            round_scores();
            if (n_full == 0) mask_scores(0);
#pragma unroll
            for (int g2 = 0; g2 < NQ; ++g2) {   // every column's first reference: its maximum in the first chunk (finite: position 0 is visible to all)
                m_ref[g2] = max_xor32(max_xor16(local_max(g2)));
#pragma unroll
                for (int j = 0; j < 4; ++j) { sA[g2][j] -= m_ref[g2]; sB[g2][j] -= m_ref[g2]; nmq[g2][j] = -m_ref[g2]; }
            }
        }
        int c = 0;
        for (; c < n_full; ++c) iter(plain, c);
        for (; c < n_own; ++c) iter(masked, c);
        // (the epilogue reads the running outputs with instructions the compiler places without knowing of the MFMAs above)
        // (every variable once: for an operand listed twice the compiler makes a copy in front, itself such an instruction)
        if constexpr (NQ == 1) asm volatile("s_nop 15\n\ts_nop 15" : "+v"(acc_o[0][DT - 1]));
        else asm volatile("s_nop 15\n\ts_nop 15" : "+v"(acc_o[0][DT - 1]), "+v"(acc_o[1][DT - 1]));
        for (int j = n_own + 1; j <= nchunks; ++j) wait_barrier(j);      // every wavefront passes barriers 0 ... nchunks
    }
    // outputs through this wavefront's LDS slice so that rows go out contiguously: O^T[d][col] -> out[row(col)][d]
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");      // (no request of this block outlives it)
    __builtin_amdgcn_s_barrier();
    if (!active) return;
    float* so = (float*)sbuf[w];              // [D / 2][16 columns]
#pragma unroll
    for (int g2 = 0; g2 < NQ; ++g2) {
        const float l_col = sum_xor32(sum_xor16(l_run[g2]));
        if (q == 0) sl[w][r16] = l_col;
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
#pragma unroll
            for (int dt = 0; dt < DT / 2; ++dt)
#pragma unroll
                for (int i = 0; i < 4; ++i) so[(dt * 16 + 4 * q + i) * 16 + r16] = acc_o[g2][hf * (DT / 2) + dt][i];
            __builtin_amdgcn_wave_barrier();
            // four lanes per column: lane (col, part) divides and writes D / 8 consecutive outputs of its column as 16-byte pieces
            const int col = lane >> 2, part = lane & 3;
            const int qi = g2 * QB + col / G, g = col % G;
            if (col / G < QB && tq0 + qi < a.Tq) {
                half_t* out = (half_t*)a.out + ((long)b * a.Tq + tq0 + qi) * a.ld_out + (kvh * G + g) * D + hf * (D / 2) + part * (D / 8);
                const float inv = 1.0f / sl[w][col];
#pragma unroll
                for (int d8 = 0; d8 < D / 8; d8 += 8) {
                    half8 o;
#pragma unroll
                    for (int j = 0; j < 8; ++j) o[j] = (half_t)(so[(part * (D / 8) + d8 + j) * 16 + col] * inv);
                    *(half8*)(out + d8) = o;
                }
            }
            __builtin_amdgcn_wave_barrier();
        }
    }
}

// ------------------------------------------------------------------------------------------------
// sampling on the device
// ------------------------------------------------------------------------------------------------
// Greedy: argmax over a row of logits, lowest index among equal maxima (TensorApplyCPU.cs:339-360 applied to the
// softmax output; softmax is monotone, so the winner is the same up to ties created by rounding of the division).
// last_pos (optional): table [rows][last_ld] of the last sequence index of every token; the chosen token is recorded
// at index *d_len (the sequence length before it is appended).
// blocked (optional): one byte per token; the reference adds -1 to the probabilities of blocked tokens
// (Decoder.cs:745-753), which puts them below every other token: they are left out here.  (A blocked token could
// only win there if every other probability had underflowed to zero.)
// (1024 threads; the chosen token is returned to every thread)
__device__ __forceinline__ int greedy_row(const float* __restrict__ logits, long ld, int V, int* __restrict__ next_ids,
                                          int* __restrict__ gen_out, const int* __restrict__ d_step,
                                          int* __restrict__ last_pos, long last_ld, const int* __restrict__ d_len,
                                          const unsigned char* __restrict__ blocked) {
    __shared__ float sv[16];
    __shared__ int si[16];
    __shared__ int s_tok;
    const int b = blockIdx.x, t = threadIdx.x;
    const float* row = logits + (long)b * ld;
    float best = -INFINITY; int bi = 0x7fffffff;
    for (int i0 = t; i0 < V; i0 += 1024 * 8) {
        float v[8];
        // (unconditional requests with clamped indices: all eight are in flight before the first comparison)
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = row[min(i0 + u * 1024, V - 1)];
        if (blocked) {
            unsigned char bl[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) bl[u] = blocked[min(i0 + u * 1024, V - 1)];
#pragma unroll
            for (int u = 0; u < 8; ++u) if (bl[u]) v[u] = -INFINITY;
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) if (i0 + u * 1024 >= V) v[u] = -INFINITY;
#pragma unroll
        for (int u = 0; u < 8; ++u) { int i = i0 + u * 1024; if (i < V && (v[u] > best || (v[u] == best && i < bi))) { best = v[u]; bi = i; } }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        float ov = __shfl_xor(best, o, 64); int oi = __shfl_xor(bi, o, 64);
        if (ov > best || (ov == best && oi < bi)) { best = ov; bi = oi; }
    }
    if ((t & 63) == 0) { sv[t >> 6] = best; si[t >> 6] = bi; }
    __syncthreads();
    if (t == 0) {
        for (int w = 1; w < 16; ++w) if (sv[w] > best || (sv[w] == best && si[w] < bi)) { best = sv[w]; bi = si[w]; }
        if (bi == 0x7fffffff) bi = 0;   // a row of NaNs: the reference's scan never moves off index 0
        next_ids[b] = bi;
        if (gen_out) gen_out[(d_step ? (long)*d_step * gridDim.x : 0) + b] = bi;
        if (last_pos) last_pos[(long)b * last_ld + bi] = *d_len;
        s_tok = bi;
    }
    __syncthreads();
    return s_tok;
}
__global__ __launch_bounds__(1024) void greedy_kernel(const float* __restrict__ logits, long ld, int V, int* __restrict__ next_ids,
                                                      int* __restrict__ gen_out, const int* __restrict__ d_step,
                                                      int* __restrict__ last_pos, long last_ld, const int* __restrict__ d_len,
                                                      const unsigned char* __restrict__ blocked) {
    greedy_row(logits, ld, V, next_ids, gen_out, d_step, last_pos, last_ld, d_len, blocked);
}
// The same, and the block goes on with what the next decode step would do first for its row: the embedding of the chosen
// token times sqrt(h), the first layer's normalisation input and its sums of squares (fn_prepare_kernel): one launch and
// one trip through memory for the token less per generated token.
template <int NPT>
__global__ __launch_bounds__(1024) void greedy_embed_kernel(const float* __restrict__ logits, long ld, int V, int* __restrict__ next_ids,
                                                            int* __restrict__ gen_out, const int* __restrict__ d_step,
                                                            int* __restrict__ last_pos, long last_ld, const int* __restrict__ d_len,
                                                            const unsigned char* __restrict__ blocked, FnPrepArgs pa) {
    const int tok = greedy_row(logits, ld, V, next_ids, gen_out, d_step, last_pos, last_ld, d_len, blocked);
    fn_prepare_row<NPT, 1024>(pa, blockIdx.x, tok, threadIdx.x);
}

}  // namespace tship
