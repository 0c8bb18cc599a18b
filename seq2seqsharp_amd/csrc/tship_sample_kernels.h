// Top-p sampling on the device: one block per row.
// Semantics of ComputeGraphTensor.TopPSample (Seq2SeqSharp/Tools/ComputeGraphTensor.cs:2305-2403) with
// repeatPenalty = 0 (pow(x, 0) = 1: no decay) and the per-row random draw supplied by the caller:
//   keep p > 0; order by p descending, equal p by ascending index (SortedDictionary<float, List<int>> walked in
//   reverse, each list in insertion order); running fp32 sum in that order, stop after the element that makes
//   acc >= topP; pick the first k with accP[k] / acc >= u.
// The order is produced by a stable least-significant-digit radix sort on the float bit pattern; the running
// sum is taken serially in fp32, so for given probabilities the chosen index is the reference's, bit for bit.
#pragma once

#include "tship_internal.h"

namespace tship {

struct TopPArgs {
    const float* in; long ld; int V;       // logits (softmax applied here) or probabilities
    int in_is_logits; float temperature;   // logits are divided by the temperature first (Decoder.cs:720-723)
    const float* uniforms;                 // [rows]
    float top_p;
    unsigned* keysA; unsigned* keysB; int* idxA; int* idxB; float* accp;   // scratch, each [rows][Vs]
    long Vs;
    int* next_ids; int* gen_out; float* out_f32;   // any of them may be null
    const int* d_step;                             // optional: uniforms and gen_out are indexed by *d_step * rows + row
};

__device__ __forceinline__ float block_max_256(float v, float* s) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    __syncthreads();
    if ((threadIdx.x & 63) == 0) s[threadIdx.x >> 6] = v;
    __syncthreads();
    return fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3]));
}

static __global__ __launch_bounds__(256) void topp_kernel(TopPArgs a) {
    __shared__ float sred[4];
    __shared__ unsigned short cnt[16][256];
    __shared__ int s_total[17];
    __shared__ int s_n;
    __shared__ float s_acc;
    __shared__ int s_pick;
    const int r = blockIdx.x, t = threadIdx.x, V = a.V;
    const float* row = a.in + (long)r * a.ld;
    unsigned* kA = a.keysA + (long)r * a.Vs; unsigned* kB = a.keysB + (long)r * a.Vs;
    int* iA = a.idxA + (long)r * a.Vs; int* iB = a.idxB + (long)r * a.Vs;
    float* accp = a.accp + (long)r * a.Vs;

    // probabilities (TensorApplyCPU.Softmax, TensorApplyCPU.cs:1230-1268), written as sort keys
    float sum = 1.0f, mx = 0.0f;
    if (a.in_is_logits) {
        float lm = -INFINITY;
        for (int i = t; i < V; i += 256) lm = fmaxf(lm, row[i] / a.temperature);
        mx = block_max_256(lm, sred);
        float ls = 0.0f;
        for (int i = t; i < V; i += 256) ls += expf(row[i] / a.temperature - mx);
        ls = wave_sum(ls);
        __syncthreads();
        if ((t & 63) == 0) sred[t >> 6] = ls;
        __syncthreads();
        sum = (sred[0] + sred[1]) + (sred[2] + sred[3]);
    }
    // each thread owns a contiguous chunk so that the scatter below is stable
    const int chunk = (V + 255) / 256, c0 = t * chunk, c1 = min(V, c0 + chunk);
    for (int i = c0; i < c1; ++i) {
        float p = a.in_is_logits ? expf(row[i] / a.temperature - mx) / sum : row[i];
        // p > 0: positive floats order like their bit patterns; descending order = ascending ~bits.
        // p <= 0 is dropped by the reference: give it the largest key so that it sorts behind every candidate.
        kA[i] = p > 0.0f ? ~__float_as_uint(p) : 0xffffffffu;
        iA[i] = i;
    }
    __syncthreads();
    for (int pass = 0; pass < 8; ++pass) {
        const int sh = pass * 4;
        unsigned short c[16];
#pragma unroll
        for (int d = 0; d < 16; ++d) c[d] = 0;
        for (int i = c0; i < c1; ++i) {
            unsigned d = (kA[i] >> sh) & 15u;
#pragma unroll
            for (int q = 0; q < 16; ++q) c[q] += (d == (unsigned)q);
        }
#pragma unroll
        for (int d = 0; d < 16; ++d) cnt[d][t] = c[d];
        __syncthreads();
        // exclusive scan over (digit major, thread minor): 16 threads scan one digit row each, then the digit totals
        if (t < 16) {
            int run = 0;
            for (int j = 0; j < 256; ++j) { int v = cnt[t][j]; cnt[t][j] = (unsigned short)run; run += v; }
            s_total[t] = run;
        }
        __syncthreads();
        if (t == 0) { int run = 0; for (int d = 0; d < 16; ++d) { int v = s_total[d]; s_total[d] = run; run += v; } }
        __syncthreads();
        int off[16];
#pragma unroll
        for (int d = 0; d < 16; ++d) off[d] = s_total[d] + cnt[d][t];
        for (int i = c0; i < c1; ++i) {
            unsigned k = kA[i]; int id = iA[i];
            unsigned d = (k >> sh) & 15u;
            int dst = 0;
#pragma unroll
            for (int q = 0; q < 16; ++q) if (d == (unsigned)q) { dst = off[q]; off[q] += 1; }
            kB[dst] = k; iB[dst] = id;
        }
        __syncthreads();
        unsigned* tk = kA; kA = kB; kB = tk;
        int* ti = iA; iA = iB; iB = ti;
    }
    // serial fp32 prefix in sorted order by the first wavefront; every lane keeps the same running value
    if (t < 64) {
        float acc = 0.0f; int n = 0; bool done = false;
        for (int base = 0; base < V && !done; base += 64) {
            int i = base + t;
            unsigned k = i < V ? kA[i] : 0xffffffffu;
            float p = k == 0xffffffffu ? 0.0f : __uint_as_float(~k);
            float mine = 0.0f;
            for (int j = 0; j < 64; ++j) {
                float pj = __shfl(p, j, 64);
                if (pj <= 0.0f) { done = true; break; }        // ran out of candidates
                acc += pj; n += 1;
                if (t == j) mine = acc;
                if (acc >= a.top_p) { done = true; break; }
            }
            if (i < V) accp[i] = mine;
        }
        if (t == 0) { s_n = n; s_acc = acc; s_pick = 0x7fffffff; }
    }
    __syncthreads();
    const long slot = (a.d_step ? (long)*a.d_step * gridDim.x : 0) + r;
    const int n = s_n; const float acc = s_acc, u = a.uniforms[slot];
    int best = 0x7fffffff;
    for (int k = t; k < n; k += 256) if (accp[k] / acc >= u) { best = k; break; }
    atomicMin(&s_pick, best);
    __syncthreads();
    if (t == 0) {
        int id = s_pick == 0x7fffffff ? 0 : iA[s_pick];
        if (a.next_ids) a.next_ids[r] = id;
        if (a.gen_out) a.gen_out[slot] = id;
        if (a.out_f32) a.out_f32[r] = (float)id;
    }
}

}  // namespace tship
