// MoE feed-forward kernels (decode-sized row counts).
// MoEFeedForward.Process, Seq2SeqSharp/Layers/MoEFeedForward.cs:76-181: LayerNorm -> router Affine -> + (-65000)
// -> Softmax -> TopK -> per-expert token lists (ascending token order) -> gather -> expert MLP -> scale by the
// expert's softmax probability -> scatter-add in expert-major order -> residual.
//
// The routing decision is index work, so the arithmetic that feeds it is done in the reference's own operation
// order: LayerNorm sums in 8-lane partial sums (TensorApplyCPU.cs:1381-1409), the router dot product serially
// over k with separately rounded product and sum (SGEMM.cs:482-549), exp evaluated in double
// (TensorApplyCPU.cs:1246), TopK by the reference's insertion rule (TensorApplyCPU.cs:1099-1146).
#pragma once

#include "tship_gpt_kernels.h"

namespace tship {

struct MoeRouterArgs {
    float* x; long ldx; int h;
    const float* part; int KS; long split_stride; long ld_part; const float* bias;   // pending attention output
    const float* gamma; const float* beta; float eps;
    const float* router; const float* router_b; int E; int k;
    float* xn32; float* probs; float* top_val; float* top_idx;
    int router_lds;      // 1: the launch reserved LDS for the router matrix
    // fast kernel only, when xg16 is set: the row's place in each chosen expert's batch is taken from the expert's counter
    // and the normalised row is written there in fp16 (fragment packed), so that no list or gather launch follows
    half_t* xg16; long xg_estride; int packed_kt; int* counts; int* slot; int max_rows;
    // fast kernel only, when xn16 is set (prefill): the normalised row leaves as fp16, row-major with ld_xn16 elements per
    // row, where the experts' up projection reads it through the token lists; xn32 is not written
    half_t* xn16; long ld_xn16;
};

__device__ __forceinline__ float tree8(float v) {
    // ((l0+l1)+(l2+l3))+((l4+l5)+(l6+l7)) across 8 adjacent lanes
    v += __shfl_xor(v, 1, 64);
    v += __shfl_xor(v, 2, 64);
    v += __shfl_xor(v, 4, 64);
    return v;
}

// One block of 256 threads per token row.  Dynamic LDS: x[h], xn[h], and the router matrix [h][E] when it fits
// (a.router_lds != 0), so that the serial dot products read LDS only.
__global__ __launch_bounds__(256) void moe_router_kernel(MoeRouterArgs a) {
#pragma clang fp contract(off)
    extern __shared__ __attribute__((aligned(16))) float moe_smem[];
    __shared__ float sr[64];
    __shared__ float s_ov[64], s_oi[64];
    __shared__ float s_stat[2];
    const int r = blockIdx.x, t = threadIdx.x, h = a.h, E = a.E;
    float* sx = moe_smem;
    float* sxn = moe_smem + h;
    float* srt = moe_smem + 2 * h;
    for (int c0 = t; c0 < h; c0 += 256 * 4) {
        float xv[4], pv[4][8], bv[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int c = c0 + u * 256;
            const bool ok = c < h;
            xv[u] = ok ? a.x[(long)r * a.ldx + c] : 0.0f;
            bv[u] = (ok && a.part) ? a.bias[c] : 0.0f;
#pragma unroll
            for (int k = 0; k < 8; ++k) pv[u][k] = (ok && a.part && k < a.KS) ? a.part[k * a.split_stride + (long)r * a.ld_part + c] : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int c = c0 + u * 256;
            if (c >= h) continue;
            float v = xv[u];
            if (a.part) {
                float s = pv[u][0];
#pragma unroll
                for (int k = 1; k < 8; ++k) if (k < a.KS) s += pv[u][k];
                for (int k = 8; k < a.KS; ++k) s += a.part[k * a.split_stride + (long)r * a.ld_part + c];
                v = (s + bv[u]) + v;
                a.x[(long)r * a.ldx + c] = v;
            }
            sx[c] = v;
        }
    }
    __syncthreads();
    // LayerNorm statistics in the reference's order (TensorApplyCPU.cs:1381-1409): eight interleaved partial sums
    // added as a tree, then the tail; for the variance every group of eight squared deviations is added as a tree and
    // the group sums sequentially.  The group trees are independent, so all threads compute them; only the two short
    // sequential chains run on one thread.
    const int ng = h > 8 ? (h - 8 + 7) / 8 : 0;       // full groups handled by the interleaved loops
    if (t < 8) {
        float lane = 0.0f;
#pragma unroll 8
        for (int j = 0; j < ng; ++j) lane += sx[8 * j + t];
        float sum = tree8(lane);
        for (int i = 8 * ng; i < h; ++i) sum += sx[i];
        if (t == 0) s_stat[0] = sum / (float)h;
    }
    __syncthreads();
    {
        const float mean0 = s_stat[0];
        for (int j = t; j < ng; j += 256) {
            float dd[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) { const float d = sx[8 * j + u] - mean0; dd[u] = d * d; }
            sxn[j] = ((dd[0] + dd[1]) + (dd[2] + dd[3])) + ((dd[4] + dd[5]) + (dd[6] + dd[7]));
        }
    }
    __syncthreads();
    if (t == 0) {
        const float mean0 = s_stat[0];
        float sq = 0.0f;
#pragma unroll 8
        for (int j = 0; j < ng; ++j) sq += sxn[j];
        for (int i = 8 * ng; i < h; ++i) { const float d = sx[i] - mean0; sq += d * d; }
        s_stat[1] = sqrtf(a.eps + sq / (float)h);
    }
    __syncthreads();
    const float mean = s_stat[0], sigma = s_stat[1];
    for (int c0 = t; c0 < h; c0 += 256 * 4) {
        float gv[4], bv[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) { const int c = c0 + u * 256; gv[u] = c < h ? a.gamma[c] : 0.0f; bv[u] = c < h ? a.beta[c] : 0.0f; }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int c = c0 + u * 256;
            if (c >= h) continue;
            float y = gv[u] * ((sx[c] - mean) / sigma);
            y += bv[u];
            sxn[c] = y;
            a.xn32[(long)r * h + c] = y;
        }
    }
    __syncthreads();
    // Router logits: sum over l of xn[l] * W[l][e], product and sum rounded separately, added strictly in order of l
    // (SGEMM.cs:482-549; rows with xn[l] == 0 are skipped there, which equals adding a zero product).  The products
    // are independent, so all threads form them (transposed into LDS: pt[e][l]); one thread per expert then adds its
    // h products in order, reading them 16 bytes at a time.
    if (a.router_lds) {
        float* pt = srt;
        const int n = h * E;
        for (int i0 = t; i0 < n; i0 += 256 * 8) {
            float wv[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) { const int i = i0 + u * 256; wv[u] = i < n ? a.router[i] : 0.0f; }
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int i = i0 + u * 256;
                if (i < n) { const int l = i / E, e = i - l * E; const float xv = sxn[l]; pt[e * h + l] = xv != 0.0f ? xv * wv[u] : 0.0f; }
            }
        }
        __syncthreads();
    }
    if (t < E) {
        float acc = a.router_b[t];
        if (a.router_lds) {
            const float* p = srt + t * h;
            int l = 0;
            if ((h & 3) == 0) {
                for (; l + 16 <= h; l += 16) {
                    floatx4 q0 = *(const floatx4*)(p + l), q1 = *(const floatx4*)(p + l + 4), q2 = *(const floatx4*)(p + l + 8), q3 = *(const floatx4*)(p + l + 12);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int u = 0; u < 4; ++u) acc += q0[u];
#pragma unroll
                    for (int u = 0; u < 4; ++u) acc += q1[u];
#pragma unroll
                    for (int u = 0; u < 4; ++u) acc += q2[u];
#pragma unroll
                    for (int u = 0; u < 4; ++u) acc += q3[u];
                }
            }
            for (; l < h; ++l) acc += p[l];
        } else {
            for (int l = 0; l < h; ++l) { const float xv = sxn[l]; if (xv != 0.0f) acc += xv * a.router[(long)l * E + t]; }
        }
        sr[t] = acc + (-65000.0f);
    }
    __syncthreads();
    // the exponentials (evaluated in double, the expensive part) do not depend on each other: one lane per expert; only
    // their sum has an order
    if (t < 64) {
        float mx = sr[0];
        for (int e = 1; e < E; ++e) mx = fmaxf(mx, sr[e]);
        const float ex = t < E ? (float)exp((double)(sr[t] - mx)) : 0.0f;
        __builtin_amdgcn_wave_barrier();
        if (t < E) sr[t] = ex;
    }
    __syncthreads();
    if (t == 0) {
        const int k = a.k;
        float sum = 0.0f;
        for (int e = 0; e < E; ++e) sum += sr[e];
        float* pr = a.probs + (long)r * E;
        for (int e = 0; e < E; ++e) { sr[e] = sr[e] / sum; pr[e] = sr[e]; }
        // (the insertion works on LDS copies: on the global arrays every step would be a memory round trip)
        float* ov = s_ov; float* oi = s_oi;
        for (int i = 0; i < k; ++i) { ov[i] = -1.70141e+38f; oi[i] = -1.70141e+38f; }
        for (int e = 0; e < E; ++e) {
            float data = sr[e];
            if (data < ov[k - 1]) continue;
            int j = k - 2;
            for (; j >= 0; --j) {
                if (data > ov[j]) { ov[j + 1] = ov[j]; oi[j + 1] = oi[j]; }
                else { ov[j + 1] = data; oi[j + 1] = (float)e; break; }
            }
            if (j < 0) { ov[0] = data; oi[0] = (float)e; }
        }
        for (int i = 0; i < k; ++i) { a.top_val[(long)r * k + i] = ov[i]; a.top_idx[(long)r * k + i] = oi[i]; }
    }
}

// v of lane `l`, the same l in every lane (a register read, no trip through the cross-lane network)
__device__ __forceinline__ float lane_value(float v, int l) { return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), l)); }

// The reference's TopK (TensorApplyCPU.cs TopK: keep the K largest by insertion, walking the row once) with the row spread
// over the lanes of a wavefront (lane e holds element e) and the K kept values in registers of every lane.  An element
// equal to the smallest kept value still enters (and takes the last place); an element equal to a larger kept value goes
// behind it.  pos = the number of kept values, among the first K - 1, that the element does not exceed.
template <int K>
__device__ __forceinline__ void topk_by_insertion(float p, int E, float (&ov)[4], float (&oi)[4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) { ov[i] = -1.70141e+38f; oi[i] = -1.70141e+38f; }
    for (int e = 0; e < E; ++e) {
        const float data = lane_value(p, e);
        if (data < ov[K - 1]) continue;
        int pos = 0;
#pragma unroll
        for (int j = 0; j < K - 1; ++j) pos += (data > ov[j]) ? 0 : 1;
#pragma unroll
        for (int i = K - 1; i >= 0; --i) {
            if (i > pos) { if (i >= 1) { ov[i] = ov[i > 0 ? i - 1 : 0]; oi[i] = oi[i > 0 ? i - 1 : 0]; } }
            else if (i == pos) { ov[i] = data; oi[i] = (float)e; }
        }
    }
}

// Sums of eight values per lane over the wavefront with ten cross-lane moves instead of forty-eight: every step halves the
// number of values a lane carries (the upper half of the lanes keeps the upper half of the values), and once one value is
// left three more steps finish it.  Afterwards lane L holds the total of value ((L >> 5) & 1) * 4 + ((L >> 4) & 1) * 2 +
// ((L >> 3) & 1).
__device__ __forceinline__ float wave_sum8(const float (&acc)[8], int lane) {
    float r4[4], r2[2];
    const bool h5 = lane & 32, h4 = lane & 16, h3 = lane & 8;
#pragma unroll
    for (int u = 0; u < 4; ++u) { const float mine = h5 ? acc[u + 4] : acc[u], other = h5 ? acc[u] : acc[u + 4]; r4[u] = mine + __shfl_xor(other, 32, 64); }
#pragma unroll
    for (int u = 0; u < 2; ++u) { const float mine = h4 ? r4[u + 2] : r4[u], other = h4 ? r4[u] : r4[u + 2]; r2[u] = mine + __shfl_xor(other, 16, 64); }
    float r1 = (h3 ? r2[1] : r2[0]) + __shfl_xor(h3 ? r2[0] : r2[1], 8, 64);
    r1 += __shfl_xor(r1, 4, 64);
    r1 += __shfl_xor(r1, 2, 64);
    r1 += __shfl_xor(r1, 1, 64);
    return r1;
}

// The same routing for fp16 models, one block of 256 threads per token row, everything requested in one memory round
// trip and reduced as trees.  An fp16 model's activations differ from the fp32 reference's by the fp16 path's rounding
// (about 1e-3), which already decides near-ties differently, so reproducing the reference's serial summation order (the
// 1024-step chains of the kernel above) buys nothing there; that kernel remains the one fp32 models use, where routing
// indices are bit-exact.  Same outputs: x updated with the pending attention output, LayerNorm in fp32, router logits
// + (-65000), softmax with the exponentials evaluated in double, TopK by the reference's insertion rule.
// Thread t works on the column groups g = t, t + 256, ... of four neighbouring columns (16-byte requests; a row of 1024
// columns is one request per tensor and thread: as 4-byte requests strided by the expert count the router matrix alone
// took 3.5 us), so hidden must be a multiple of four.  With xg16 set (decode steps) the kernel also gives the row its
// place in each chosen expert's batch and writes it there (see MoeRouterArgs).
template <int NG>      // NG * 1024 >= hidden
__global__ __launch_bounds__(256) void moe_router_fast_kernel(MoeRouterArgs a) {
    constexpr int MAXE = 64;
    __shared__ float sred[4];
    __shared__ float swe[4][MAXE];
    __shared__ float sr[MAXE];
    __shared__ float s_ov[MAXE], s_oi[MAXE];
    __shared__ int s_slot[MAXE];
    const int r = blockIdx.x, t = threadIdx.x, h = a.h, E = a.E, lane = t & 63, w = t >> 6;
    floatx4 v[NG], g[NG], bt[NG];
    floatx4 wv0[NG][4][2];       // router weights of experts 0-7 for the thread's columns (E == 8: 32 bytes per column)
    const bool e8 = E == 8;
#pragma unroll
    for (int i = 0; i < NG; ++i) {
        const int c = 4 * (t + i * 256);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            if (e8 && c < h) {
                const floatx4* src = (const floatx4*)(a.router + (long)(c + q) * 8);
                wv0[i][q][0] = src[0]; wv0[i][q][1] = src[1];
            } else {
#pragma unroll
                for (int u = 0; u < 8; ++u) wv0[i][q][u >> 2][u & 3] = (c < h && u < E) ? a.router[(long)(c + q) * E + u] : 0.0f;
            }
        }
    }
    {
        floatx4 xv[NG], bv[NG], pv[NG][8];       // up to eight split-K partials requested at once
        const floatx4 zero4 = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int i = 0; i < NG; ++i) {
            const int c = 4 * (t + i * 256); const bool ok = c < h;
            xv[i] = ok ? *(const floatx4*)(a.x + (long)r * a.ldx + c) : zero4;
            bv[i] = (ok && a.part) ? *(const floatx4*)(a.bias + c) : zero4;
#pragma unroll
            for (int k = 0; k < 8; ++k) pv[i][k] = (ok && a.part && k < a.KS) ? *(const floatx4*)(a.part + k * a.split_stride + (long)r * a.ld_part + c) : zero4;
            g[i] = ok ? *(const floatx4*)(a.gamma + c) : zero4; bt[i] = ok ? *(const floatx4*)(a.beta + c) : zero4;
        }
#pragma unroll
        for (int i = 0; i < NG; ++i) {
            const int c = 4 * (t + i * 256);
            v[i] = xv[i];
            if (a.part && c < h) {
                floatx4 s = pv[i][0];
#pragma unroll
                for (int k = 1; k < 8; ++k) if (k < a.KS) s += pv[i][k];
                for (int k = 8; k < a.KS; ++k) s += *(const floatx4*)(a.part + k * a.split_stride + (long)r * a.ld_part + c);
                v[i] = (s + bv[i]) + xv[i];
                *(floatx4*)(a.x + (long)r * a.ldx + c) = v[i];
            }
        }
    }
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < NG; ++i) sum += (v[i][0] + v[i][1]) + (v[i][2] + v[i][3]);          // (columns beyond h hold zeros)
    const float mean = block_sum_256(sum, sred) / (float)h;
    float d2 = 0.0f;
#pragma unroll
    for (int i = 0; i < NG; ++i) {
        if (4 * (t + i * 256) < h) {
#pragma unroll
            for (int q = 0; q < 4; ++q) { const float d = v[i][q] - mean; d2 += d * d; }
        }
    }
    const float sigma = sqrtf(a.eps + block_sum_256(d2, sred) / (float)h);
    floatx4 y[NG];
#pragma unroll
    for (int i = 0; i < NG; ++i) {
        const int c = 4 * (t + i * 256);
#pragma unroll
        for (int q = 0; q < 4; ++q) y[i][q] = c < h ? g[i][q] * ((v[i][q] - mean) / sigma) + bt[i][q] : 0.0f;
        if (c < h && a.xn16) {
            half4 hv = {(half_t)y[i][0], (half_t)y[i][1], (half_t)y[i][2], (half_t)y[i][3]};
            *(half4*)(a.xn16 + (long)r * a.ld_xn16 + c) = hv;
        } else if (c < h && !a.xg16) *(floatx4*)(a.xn32 + (long)r * h + c) = y[i];
    }
    // router logits: every thread's columns against all experts, then a tree over the block
    for (int e0 = 0; e0 < E; e0 += 8) {
        float acc[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) acc[u] = 0.0f;
#pragma unroll
        for (int i = 0; i < NG; ++i) {
            const int c = 4 * (t + i * 256);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const float wgt = e0 == 0 ? wv0[i][q][u >> 2][u & 3] : ((c < h && e0 + u < E) ? a.router[(long)(c + q) * E + e0 + u] : 0.0f);
                    acc[u] += y[i][q] * wgt;
                }
            }
        }
        const float tot = wave_sum8(acc, lane);
        const int eu = ((lane >> 5) & 1) * 4 + ((lane >> 4) & 1) * 2 + ((lane >> 3) & 1);
        if ((lane & 7) == 0 && e0 + eu < E) swe[w][e0 + eu] = tot;
    }
    __syncthreads();
    if (a.k <= 4) {
        // softmax and TopK inside the first wavefront, in registers: lane e holds expert e, the serial steps of the reference
        // (the sum in expert order, the insertion rule) run on all lanes alike with the values read across lanes
        if (t < 64) {
            float lg = -INFINITY;
            if (t < E) lg = ((((swe[0][t] + swe[1][t]) + swe[2][t]) + swe[3][t]) + a.router_b[t]) + (-65000.0f);
            const float mx = wave_max(lg);
            const float ex = t < E ? (float)exp((double)(lg - mx)) : 0.0f;
            float ssum = 0.0f;
            for (int e = 0; e < E; ++e) ssum += lane_value(ex, e);
            const float p = ex / ssum;
            if (t < E) a.probs[(long)r * E + t] = p;
            float ov[4], oi[4];
            switch (a.k) {
                case 1: topk_by_insertion<1>(p, E, ov, oi); break;
                case 2: topk_by_insertion<2>(p, E, ov, oi); break;
                case 3: topk_by_insertion<3>(p, E, ov, oi); break;
                default: topk_by_insertion<4>(p, E, ov, oi); break;
            }
            if (t == 0) {
                const int k = a.k;
#pragma unroll
                for (int i = 0; i < 4; ++i) if (i < k) { a.top_val[(long)r * k + i] = ov[i]; a.top_idx[(long)r * k + i] = oi[i]; s_oi[i] = oi[i]; }
                if (a.xg16) {
                    // The row's place in each chosen expert's batch: the order in which rows arrive differs from run to run,
                    // the results do not (a row's product does not depend on its place, and the combine step adds a token's
                    // experts in expert order whatever their places).  The counters are zero on entry: the combine kernel
                    // clears them.  All requests go out before the first answer is needed.
                    int sl[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) sl[i] = i < k ? (int)__hip_atomic_fetch_add(a.counts + (int)oi[i], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0;
#pragma unroll
                    for (int i = 0; i < 4; ++i) if (i < k) { s_slot[i] = sl[i]; a.slot[(long)r * k + i] = sl[i]; }
                }
            }
        }
    } else {
        if (t < 64) {
            float lg = -INFINITY;
            if (t < E) lg = ((((swe[0][t] + swe[1][t]) + swe[2][t]) + swe[3][t]) + a.router_b[t]) + (-65000.0f);
            const float mx = wave_max(lg);
            const float ex = t < E ? (float)exp((double)(lg - mx)) : 0.0f;
            if (t < E) sr[t] = ex;
        }
        __syncthreads();
        if (t == 0) {
            const int k = a.k;
            float s = 0.0f;
            for (int e = 0; e < E; ++e) s += sr[e];
            float* pr = a.probs + (long)r * E;
            for (int e = 0; e < E; ++e) { sr[e] = sr[e] / s; pr[e] = sr[e]; }
            // (the insertion works on LDS copies: on the global arrays every step would be a memory round trip)
            float* ov = s_ov; float* oi = s_oi;
            for (int i = 0; i < k; ++i) { ov[i] = -1.70141e+38f; oi[i] = -1.70141e+38f; }
            for (int e = 0; e < E; ++e) {
                float data = sr[e];
                if (data < ov[k - 1]) continue;
                int j = k - 2;
                for (; j >= 0; --j) {
                    if (data > ov[j]) { ov[j + 1] = ov[j]; oi[j + 1] = oi[j]; }
                    else { ov[j + 1] = data; oi[j + 1] = (float)e; break; }
                }
                if (j < 0) { ov[0] = data; oi[0] = (float)e; }
            }
            for (int i = 0; i < k; ++i) { a.top_val[(long)r * k + i] = ov[i]; a.top_idx[(long)r * k + i] = oi[i]; }
            if (a.xg16) {
                for (int i = 0; i < k; ++i) {
                    const int sl = (int)__hip_atomic_fetch_add(a.counts + (int)oi[i], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    s_slot[i] = sl; a.slot[(long)r * k + i] = sl;
                }
            }
        }
    }
    if (a.xg16) {
        __syncthreads();
        for (int i = 0; i < a.k; ++i) {
            half_t* dst = a.xg16 + (long)(int)s_oi[i] * a.xg_estride;
            const int sl = s_slot[i];
            if (sl >= a.max_rows) continue;
#pragma unroll
            for (int q = 0; q < NG; ++q) {
                const int c = 4 * (t + q * 256);
                if (c < h) {
                    half4 hv = {(half_t)y[q][0], (half_t)y[q][1], (half_t)y[q][2], (half_t)y[q][3]};
                    *(half4*)(dst + xpack_index(sl, c, a.packed_kt)) = hv;       // (four neighbouring columns are neighbours in a fragment)
                }
            }
        }
    }
}

// per-expert token lists in ascending token order (MoEFeedForward.cs:92-105); slot[i*k+j] = position of token i in
// the list of its j-th expert
__global__ __launch_bounds__(64) void moe_lists_kernel(const float* __restrict__ top_idx, int rows, int k, int E, int max_rows, int* __restrict__ counts,
                                                        int* __restrict__ lists, int* __restrict__ slot) {
    extern __shared__ int s_idx[];
    for (int i = threadIdx.x; i < rows * k; i += 64) s_idx[i] = (int)top_idx[i];
    __syncthreads();
    int e = threadIdx.x;
    if (e >= E) return;
    int n = 0;
    for (int i = 0; i < rows * k; ++i)
        if (s_idx[i] == e) { lists[e * max_rows + n] = i / k; slot[i] = n; ++n; }
    counts[e] = n;
}

// The same lists for many rows (prefill): one block of 1024 threads per expert walks the (token, choice) pairs in order,
// 1024 at a time; a pair's place in the list is the number of the expert's pairs before it (ballots inside a wavefront,
// wavefront totals through LDS), so the lists come out in ascending token order like the serial kernel's.
__global__ __launch_bounds__(1024) void moe_lists_big_kernel(const float* __restrict__ top_idx, int rows, int k, int max_rows, int* __restrict__ counts,
                                                              int* __restrict__ lists, int* __restrict__ slot) {
    __shared__ int s_wave[2][16];
    const int e = blockIdx.x, t = threadIdx.x, lane = t & 63, w = t >> 6;
    const int n_pairs = rows * k;
    int base = 0;            // the expert's pairs before this round (every thread keeps its own copy)
    // a thread takes four consecutive pairs per round (4096 pairs per round and block); the rounds alternate between
    // two sets of wavefront totals, so one barrier per round is enough
    int par = 0;
    for (int i0 = 0; i0 < n_pairs; i0 += 4096, par ^= 1) {
        const int i = i0 + 4 * t;
        float tv[4];
        if (i + 3 < n_pairs) { const floatx4 q = *(const floatx4*)(top_idx + i); tv[0] = q[0]; tv[1] = q[1]; tv[2] = q[2]; tv[3] = q[3]; }
        else {
#pragma unroll
            for (int j = 0; j < 4; ++j) tv[j] = i + j < n_pairs ? top_idx[i + j] : -1.0f;
        }
        bool hit[4];
        int before = 0, total = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            hit[j] = (int)tv[j] == e;
            const unsigned long long bal = __ballot(hit[j]);
            before += __popcll(bal & ((1ull << lane) - 1ull));          // the lower lanes' pairs all come first
            total += __popcll(bal);
        }
        if (lane == 0) s_wave[par][w] = total;
        __syncthreads();
        int off = base, all = 0;
#pragma unroll
        for (int j = 0; j < 16; ++j) { const int c = s_wave[par][j]; off += j < w ? c : 0; all += c; }
        int n = off + before;
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (hit[j]) { lists[(long)e * max_rows + n] = (i + j) / k; slot[i + j] = n; ++n; }
        base += all;
    }
    if (t == 0) counts[e] = base;
}

// rows row_map[b] of up to three [.., width] tables -> rows b of others (the routing of each sequence's last prompt
// position, kept where the decode step keeps its routing): grid (batch, tables)
struct MoeRowsArgs { const float* src[3]; float* dst[3]; int width[3]; const int* row_map; };
__global__ void moe_rows_kernel(MoeRowsArgs a) {
    const int b = blockIdx.x, q = blockIdx.y;
    const float* src = a.src[q]; float* dst = a.dst[q]; const int width = a.width[q];
    for (int c = threadIdx.x; c < width; c += blockDim.x) dst[(long)b * width + c] = src[(long)a.row_map[b] * width + c];
}

// IndexSelect(inputNorm, tokenIdx_e) for every expert (MoEFeedForward.cs:155): grid (max_rows, E)
template <typename AT>
__global__ __launch_bounds__(256) void moe_gather_kernel(const float* __restrict__ xn32, int h, const int* __restrict__ counts,
                                                          const int* __restrict__ lists, int max_rows, AT* __restrict__ xg, long ld, long estride,
                                                          int packed_kt) {
    const int j = blockIdx.x, e = blockIdx.y;
    if (j >= counts[e]) return;
    const int tok = lists[e * max_rows + j];
    AT* dst = xg + e * estride;
    for (int c = threadIdx.x; c < h; c += 256) {
        if (packed_kt > 0) dst[xpack_index(j, c, packed_kt)] = (AT)xn32[(long)tok * h + c];
        else dst[(long)j * ld + c] = (AT)xn32[(long)tok * h + c];
    }
}

// Lists and gather in one launch for decode-sized batches (at most 1024 (token, choice) pairs): block (j, e) finds the
// j-th pair of expert e by itself (every block repeats the small ordered count: ballots inside a wavefront, wavefront
// totals through LDS, pairs t, t + 256, ... in four rounds), records the pair's slot, and copies the token's row.
// Block (0, e) stores the expert's count.  Same lists, same order as moe_lists_kernel.
template <typename AT>
__global__ __launch_bounds__(256) void moe_gather_lists_kernel(const float* __restrict__ top_idx, int rows, int k, const float* __restrict__ xn32, int h,
                                                                int* __restrict__ counts, int* __restrict__ lists, int* __restrict__ slot, int max_rows,
                                                                AT* __restrict__ xg, long ld, long estride, int packed_kt) {
    __shared__ int s_wave[4];
    __shared__ int s_pair;
    const int j = blockIdx.x, e = blockIdx.y, t = threadIdx.x, lane = t & 63, w = t >> 6;
    const int n_pairs = rows * k;
    if (t == 0) s_pair = -1;
    int base = 0;
    for (int q = 0; q < 4; ++q) {
        const int i = q * 256 + t;
        const bool hit = i < n_pairs && (int)top_idx[i] == e;
        const unsigned long long bal = __ballot(hit);
        const int before = __popcll(bal & ((1ull << lane) - 1ull));
        __syncthreads();                       // (s_wave of the round before has been read)
        if (lane == 0) s_wave[w] = __popcll(bal);
        __syncthreads();
        int off = base;
        for (int x = 0; x < w; ++x) off += s_wave[x];
        if (hit && off + before == j) s_pair = i;
        base += s_wave[0] + s_wave[1] + s_wave[2] + s_wave[3];
    }
    __syncthreads();
    if (j == 0 && t == 0) counts[e] = base;
    const int pair = s_pair;
    if (pair < 0) return;                      // fewer than j + 1 tokens chose this expert
    const int tok = pair / k;
    if (t == 0) { slot[pair] = j; lists[e * max_rows + j] = tok; }
    AT* dst = xg + e * estride;
    for (int c = t; c < h; c += 256) {
        if (packed_kt > 0) dst[xpack_index(j, c, packed_kt)] = (AT)xn32[(long)tok * h + c];
        else dst[(long)j * ld + c] = (AT)xn32[(long)tok * h + c];
    }
}

// EltMul by the expert's probability, scatter-add in expert-major order into zeros, then input + result
// (MoEFeedForward.cs:167-178; IndexSelectGrad, TensorApplyCPU.cs:1336-1356): one block per token
__global__ __launch_bounds__(256) void moe_combine_kernel(float* __restrict__ x, long ldx, int h, const float* __restrict__ y, long ldy, long estride,
                                                           const float* __restrict__ probs, const float* __restrict__ top_idx, const int* __restrict__ slot,
                                                           int k, int E, int* __restrict__ clear_counts) {
#pragma clang fp contract(off)
    const int i = blockIdx.x;
    if (clear_counts && i == 0 && (int)threadIdx.x < E) clear_counts[threadIdx.x] = 0;       // for the next router launch
    if (k <= 8 && h % 4 == 0 && ldx % 4 == 0 && ldy % 4 == 0 && estride % 4 == 0) {
        // The token's picks in expert-major order (equal experts in pick order), found once per thread instead of once
        // per element and expert; then the same products and sums in that order, four columns per thread and request.
        int ex[8], sl[8]; float pr[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int jj = min(j, k - 1);
            ex[j] = j < k ? (int)top_idx[i * k + jj] : 0x7fffffff;
            sl[j] = slot[i * k + jj];
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) pr[j] = j < k ? probs[i * E + min(max(ex[j], 0), E - 1)] : 0.0f;
        int ord[8];          // ord[r] = pick with rank r
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            int rank = 0;
#pragma unroll
            for (int o = 0; o < 8; ++o) rank += (ex[o] < ex[j] || (ex[o] == ex[j] && o < j)) ? 1 : 0;
#pragma unroll
            for (int r = 0; r < 8; ++r) if (r == rank) ord[r] = j;
        }
        for (int c = 4 * threadIdx.x; c < h; c += 1024) {
            floatx4 yv[8];
#pragma unroll
            for (int r = 0; r < 8; ++r) {
                // (pick number ord[r], selected without dynamic register indexing)
                int e = 0, s_ = 0;
#pragma unroll
                for (int j = 0; j < 8; ++j) if (ord[r] == j) { e = ex[j]; s_ = sl[j]; }
                const bool on = r < k && e >= 0 && e < E;
                yv[r] = on ? *(const floatx4*)(y + (long)e * estride + (long)s_ * ldy + c) : floatx4{0.0f, 0.0f, 0.0f, 0.0f};
            }
            floatx4 xv = *(const floatx4*)(x + (long)i * ldx + c);
            floatx4 out = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int r = 0; r < 8; ++r) {
                float p = 0.0f; int e = -1;
#pragma unroll
                for (int j = 0; j < 8; ++j) if (ord[r] == j) { p = pr[j]; e = ex[j]; }
                if (r < k && e >= 0 && e < E) {
#pragma unroll
                    for (int q = 0; q < 4; ++q) { const float sc = yv[r][q] * p; out[q] += sc; }
                }
            }
#pragma unroll
            for (int q = 0; q < 4; ++q) xv[q] = xv[q] + out[q];
            *(floatx4*)(x + (long)i * ldx + c) = xv;
        }
        return;
    }
    for (int c = threadIdx.x; c < h; c += 256) {
        float out = 0.0f;
        for (int e = 0; e < E; ++e)
            for (int j = 0; j < k; ++j)
                if ((int)top_idx[i * k + j] == e) {
                    float sc = y[e * estride + (long)slot[i * k + j] * ldy + c] * probs[i * E + e];
                    out += sc;
                }
        x[(long)i * ldx + c] = x[(long)i * ldx + c] + out;
    }
}

}  // namespace tship
