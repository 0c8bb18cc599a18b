// Top-p sampling on the device.
// Semantics of ComputeGraphTensor.TopPSample (Seq2SeqSharp/Tools/ComputeGraphTensor.cs:2305-2403) with the per-row
// random draw supplied by the caller:
//   keep p > 0; a token that occurs in the row's sequence so far is decayed,
//   p = (float)(p * (float)pow((float)dist / (float)len, repeatPenalty)), dist = len - (index of its last occurrence)
//   (:2320-2345; the sequence is prompt + generated tokens, Decoder.cs:761); order by p descending, equal p by
//   ascending index (SortedDictionary<float, List<int>> walked in reverse, each list in insertion order); running
//   fp32 sum in that order, stop after the element that makes acc >= topP; pick the first k with accP[k] / acc >= u.
// The last occurrence of every token is kept in a table [rows][vocabulary] (-1: not in the sequence) that the
// caller maintains (history_kernel for given tokens; the pick and greedy kernels record the token they choose).
// The order is produced by a stable least-significant-digit radix sort on the float bit pattern (four passes of
// eight bits, every pass = histogram, scan, scatter over segments of 1024 elements, so a row is sorted by many
// blocks); the running sum is taken serially in fp32 by one wavefront, so for given probabilities the chosen index
// is the reference's, bit for bit.
#pragma once

#include "tship_internal.h"

namespace tship {

constexpr int TOPP_SEG = 1024;            // elements per sort block: 4 wavefronts x 4 rounds x 64 lanes, in index order

struct TopPArgs {
    const float* in; long ld; int V;       // logits (softmax applied here) or probabilities
    int in_is_logits; float temperature;   // logits are divided by the temperature first (Decoder.cs:720-723)
    const float* uniforms;                 // [rows]
    float top_p;
    unsigned* keysA; unsigned* keysB; int* idxA; int* idxB; float* accp;   // scratch, each [rows][Vs]
    long Vs;
    int* hist; int nseg;                   // scratch [rows][nseg][256]
    int shift;                             // digit of the current sort pass
    int* next_ids; int* gen_out; float* out_f32;   // any of them may be null
    const int* d_step;                             // optional: uniforms and gen_out are indexed by *d_step * rows + row
    // repeat penalty (0: none).  last_pos [rows][last_ld]; the row's sequence length is row_lens[row], else *d_len,
    // else len.  record != 0: the pick kernel stores the chosen token's index (= that length) into the table.
    float repeat_penalty; int* last_pos; long last_ld; const int* row_lens; const int* d_len; int len; int record;
    // one byte per token, non-zero = blocked: the reference adds -1 to such a probability (Decoder.cs:745-753), so it is
    // <= 0 and never a candidate.  May be null.
    const unsigned char* blocked;
};

__device__ __forceinline__ int topp_seq_len(const TopPArgs& a, int r) { return a.row_lens ? a.row_lens[r] : (a.d_len ? *a.d_len : a.len); }

// last occurrence of every token of `ids` [rows][Tq] (sequence indices pos0 .. pos0 + Tq - 1, or fewer per row when
// row_lens is given): grid (ceil(rows Tq / 256)), 256 threads
static __global__ __launch_bounds__(256) void history_kernel(const int* __restrict__ ids, int rows, int Tq, long ld_ids, int pos0, const int* __restrict__ row_lens,
                                                             int V, int* __restrict__ last_pos, long last_ld) {
    const long idx = (long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (long)rows * Tq) return;
    const int r = (int)(idx / Tq), j = (int)(idx % Tq);
    if (row_lens && j >= row_lens[r]) return;
    const int tok = ids[(long)r * ld_ids + j];
    if (tok >= 0 && tok < V) atomicMax(&last_pos[(long)r * last_ld + tok], pos0 + j);
}

inline size_t topp_scratch_bytes(long rows, long V) {
    const long Vs = round_up(V, 64), nseg = ceil_div(V, (long)TOPP_SEG);
    return (size_t)rows * Vs * 5 * 4 + (size_t)rows * nseg * 256 * 4;
}
inline void topp_carve(TopPArgs& a, void* scratch, long rows, long V) {
    const long Vs = round_up(V, 64);
    char* s = (char*)scratch; const size_t one = (size_t)rows * Vs * 4;
    a.Vs = Vs; a.nseg = (int)ceil_div(V, (long)TOPP_SEG);
    a.keysA = (unsigned*)s; a.keysB = (unsigned*)(s + one); a.idxA = (int*)(s + 2 * one); a.idxB = (int*)(s + 3 * one);
    a.accp = (float*)(s + 4 * one); a.hist = (int*)(s + 5 * one);
}

__device__ __forceinline__ float block_max_256(float v, float* s) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    __syncthreads();
    if ((threadIdx.x & 63) == 0) s[threadIdx.x >> 6] = v;
    __syncthreads();
    return fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3]));
}

__device__ __forceinline__ float block_max_1024(float v, float* s) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    __syncthreads();
    if ((threadIdx.x & 63) == 0) s[threadIdx.x >> 6] = v;
    __syncthreads();
    float m = s[0];
#pragma unroll
    for (int i = 1; i < 16; ++i) m = fmaxf(m, s[i]);
    return m;
}

// probabilities (TensorApplyCPU.Softmax, TensorApplyCPU.cs:1230-1268) written as sort keys: grid (rows), 1024 threads
static __global__ __launch_bounds__(1024) void topp_keys_kernel(TopPArgs a) {
    __shared__ float sred[16];
    const int r = blockIdx.x, t = threadIdx.x, V = a.V;
    const float* row = a.in + (long)r * a.ld;
    unsigned* kA = a.keysA + (long)r * a.Vs;
    int* iA = a.idxA + (long)r * a.Vs;
    float sum = 1.0f, mx = 0.0f;
    if (a.in_is_logits) {
        float lm = -INFINITY;
        for (int i = t; i < V; i += 1024) lm = fmaxf(lm, row[i] / a.temperature);
        mx = block_max_1024(lm, sred);
        float ls = 0.0f;
        for (int i = t; i < V; i += 1024) ls += expf(row[i] / a.temperature - mx);
        ls = wave_sum(ls);
        __syncthreads();
        if ((t & 63) == 0) sred[t >> 6] = ls;
        __syncthreads();
        sum = 0.0f;
#pragma unroll
        for (int i = 0; i < 16; ++i) sum += sred[i];
    }
    const bool decay = a.last_pos && a.repeat_penalty != 0.0f;
    const int len = decay ? topp_seq_len(a, r) : 0;
    const int* last = decay ? a.last_pos + (long)r * a.last_ld : nullptr;
    for (int i = t; i < V; i += 1024) {
        float p = a.in_is_logits ? expf(row[i] / a.temperature - mx) / sum : row[i];
        if (decay && p > 0.0f) {
            const int lp = last[i];
            if (lp >= 0) {
                // float division, double pow, one rounding to float, one fp32 multiply (ComputeGraphTensor.cs:2341-2342)
                const float ratio = (float)(len - lp) / (float)len;
                const float rp = (float)pow((double)ratio, (double)a.repeat_penalty);
                p = p * rp;      // (a product that underflows to 0 stays a candidate of weight 0 there; it can never be picked)
            }
        }
        // p > 0: positive floats order like their bit patterns; descending order = ascending ~bits.
        // p <= 0 is dropped by the reference: give it the largest key so that it sorts behind every candidate.
        kA[i] = (p > 0.0f && !(a.blocked && a.blocked[i])) ? ~__float_as_uint(p) : 0xffffffffu;
        iA[i] = i;
    }
}

// digit counts of one segment: grid (nseg, rows), 256 threads
static __global__ __launch_bounds__(256) void topp_hist_kernel(TopPArgs a) {
    __shared__ int h[256];
    const int seg = blockIdx.x, r = blockIdx.y, t = threadIdx.x;
    const unsigned* k = a.keysA + (long)r * a.Vs;
    h[t] = 0;
    __syncthreads();
#pragma unroll
    for (int it = 0; it < 4; ++it) {
        const int e = seg * TOPP_SEG + it * 256 + t;
        if (e < a.V) atomicAdd(&h[(k[e] >> a.shift) & 255u], 1);
    }
    __syncthreads();
    a.hist[((long)r * a.nseg + seg) * 256 + t] = h[t];
}

// exclusive scan in (digit major, segment minor) order: grid (rows), 256 threads (one digit each)
static __global__ __launch_bounds__(256) void topp_scan_kernel(TopPArgs a) {
    __shared__ int tot[256];
    const int r = blockIdx.x, d = threadIdx.x;
    int* h = a.hist + (long)r * a.nseg * 256;
    // (loads in batches of eight: a load-modify-store loop would wait for memory once per segment)
    int run = 0;
    for (int s0 = 0; s0 < a.nseg; s0 += 8) {
        int v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = s0 + u < a.nseg ? h[(s0 + u) * 256 + d] : 0;
#pragma unroll
        for (int u = 0; u < 8; ++u) { if (s0 + u < a.nseg) h[(s0 + u) * 256 + d] = run; run += v[u]; }
    }
    tot[d] = run;
    __syncthreads();
    if (d < 64) {       // one wavefront: 4 digits per lane, then a shuffle scan over the lane sums
        const int v0 = tot[4 * d], v1 = tot[4 * d + 1], v2 = tot[4 * d + 2], v3 = tot[4 * d + 3];
        const int mine = v0 + v1 + v2 + v3;
        int inc = mine;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) { const int n = __shfl_up(inc, o, 64); if (d >= o) inc += n; }
        const int base = inc - mine;
        tot[4 * d] = base; tot[4 * d + 1] = base + v0; tot[4 * d + 2] = base + v0 + v1; tot[4 * d + 3] = base + v0 + v1 + v2;
    }
    __syncthreads();
    const int base = tot[d];
    for (int s0 = 0; s0 < a.nseg; s0 += 8) {
        int v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = s0 + u < a.nseg ? h[(s0 + u) * 256 + d] : 0;
#pragma unroll
        for (int u = 0; u < 8; ++u) if (s0 + u < a.nseg) h[(s0 + u) * 256 + d] = v[u] + base;
    }
}

// stable scatter of one segment: grid (nseg, rows), 256 threads.  Element order inside the segment is
// (wavefront, round, lane); equal digits keep that order: rank inside a round from ballots, rounds and wavefronts
// through a prefix over their digit counts.
static __global__ __launch_bounds__(256) void topp_scatter_kernel(TopPArgs a) {
    __shared__ int wh[16][256];
    const int seg = blockIdx.x, r = blockIdx.y, t = threadIdx.x, lane = t & 63, w = t >> 6;
    const unsigned* kin = a.keysA + (long)r * a.Vs; const int* iin = a.idxA + (long)r * a.Vs;
    unsigned* kout = a.keysB + (long)r * a.Vs; int* iout = a.idxB + (long)r * a.Vs;
    for (int i = t; i < 16 * 256; i += 256) (&wh[0][0])[i] = 0;
    __syncthreads();
    unsigned key[4]; int idx[4], rank[4]; bool valid[4];
    const unsigned long long lt = (1ull << lane) - 1ull;
#pragma unroll
    for (int it = 0; it < 4; ++it) {
        const int e = seg * TOPP_SEG + w * 256 + it * 64 + lane;
        valid[it] = e < a.V;
        key[it] = valid[it] ? kin[e] : 0u;
        idx[it] = valid[it] ? iin[e] : 0;
        const unsigned d = (key[it] >> a.shift) & 255u;
        unsigned long long peers = __ballot(valid[it]);
#pragma unroll
        for (int b = 0; b < 8; ++b) {
            const bool bit = (d >> b) & 1u;
            const unsigned long long bal = __ballot(bit);
            peers &= bit ? bal : ~bal;
        }
        rank[it] = __popcll(peers & lt);
        if (valid[it] && rank[it] == 0) wh[w * 4 + it][d] = __popcll(peers);
    }
    __syncthreads();
    {
        int run = a.hist[((long)r * a.nseg + seg) * 256 + t];
#pragma unroll
        for (int s = 0; s < 16; ++s) { const int v = wh[s][t]; wh[s][t] = run; run += v; }
    }
    __syncthreads();
#pragma unroll
    for (int it = 0; it < 4; ++it) {
        if (!valid[it]) continue;
        const unsigned d = (key[it] >> a.shift) & 255u;
        const int dst = wh[w * 4 + it][d] + rank[it];
        kout[dst] = a.shift == 24 ? ~key[it] : key[it];      // the last pass leaves the probabilities' own bit patterns
        iout[dst] = idx[it];
    }
}

// running sum and pick: grid (rows), one wavefront.  keysA holds the sorted probabilities (their bit patterns, 0 for
// dropped entries), idxA the token ids in the same order.
// The running sum is one dependent chain of fp32 additions (that is what fixes its value), so the cost per element is
// what matters: the probabilities are staged through LDS in segments of 8192 (the next segment's loads are in flight
// while the current one is walked), read back 16 bytes at a time with every lane at the same address, one unit of 32
// ahead, and added with one v_add_f32 each.  The value after each unit is kept, so that the pick only replays one unit.
static __global__ __launch_bounds__(64) void topp_pick_kernel(TopPArgs a) {
    constexpr int SEG = 8192;
    __shared__ __attribute__((aligned(16))) float sp[2][SEG];
    const int r = blockIdx.x, lane = threadIdx.x, V = a.V;
    const float* pk = (const float*)(a.keysA + (long)r * a.Vs);      // Vs is a multiple of 64
    const int* idx = a.idxA + (long)r * a.Vs;
    float* cp = a.accp + (long)r * a.Vs;                               // cp[u]: running sum after unit u
    float acc = 0.0f; int n = 0, nun = 0;
    const int nseg = (V + SEG - 1) / SEG;
    floatx4 reg[SEG / 256];
    auto seg_load = [&](int s) {
#pragma unroll
        for (int i = 0; i < SEG / 256; ++i) {
            const int e = s * SEG + (i * 64 + lane) * 4;
            floatx4 v = e < V ? *(const floatx4*)(pk + e) : floatx4{0.0f, 0.0f, 0.0f, 0.0f};      // e + 3 < Vs
#pragma unroll
            for (int j = 0; j < 4; ++j) if (e + j >= V) v[j] = 0.0f;                                 // padding is not a candidate
            reg[i] = v;
        }
    };
    auto seg_store = [&](int buf) {
#pragma unroll
        for (int i = 0; i < SEG / 256; ++i) *(floatx4*)&sp[buf][(i * 64 + lane) * 4] = reg[i];
    };
    auto unit_read = [&](int buf, int u, floatx4 (&q)[8]) {
#pragma unroll
        for (int i = 0; i < 8; ++i) q[i] = *(const floatx4*)&sp[buf][u * 32 + 4 * i];
    };
    seg_load(0);
    seg_store(0);
    bool over = false;
    for (int s = 0; s < nseg && !over; ++s) {
        const int buf = s & 1;
        if (s + 1 < nseg) seg_load(s + 1);
        __builtin_amdgcn_wave_barrier();
        const int units = min(SEG, V - s * SEG + 31) / 32;             // units of this segment that hold candidates or padding
        floatx4 q[8], qn[8];
        unit_read(buf, 0, q);
        for (int u = 0; u < units; ++u) {
            if (u + 1 < units) unit_read(buf, u + 1, qn);
            // descending probabilities: candidates (p > 0) first, dropped entries and padding (0) last
            bool done = q[7][3] == 0.0f;
            if (!done) {
                float trial = acc;
#pragma unroll
                for (int i = 0; i < 8; ++i)
#pragma unroll
                    for (int j = 0; j < 4; ++j) trial += q[i][j];
                if (trial < a.top_p) { acc = trial; n += 32; }
                else done = true;
            }
            if (done) {
                // the unit that ends the walk: element by element
                for (int j = 0; j < 32; ++j) {
                    const float pj = sp[buf][u * 32 + j];
                    if (pj <= 0.0f) break;                 // ran out of candidates
                    acc += pj; n += 1;
                    if (acc >= a.top_p) break;
                }
            }
            if (lane == 0) cp[nun] = acc;
            ++nun;
            if (done) { over = true; break; }
#pragma unroll
            for (int i = 0; i < 8; ++i) q[i] = qn[i];
        }
        if (!over && s + 1 < nseg) { __builtin_amdgcn_wave_barrier(); seg_store(buf ^ 1); }
    }
    __threadfence_block();
    const long slot = (a.d_step ? (long)*a.d_step * gridDim.x : 0) + r;
    const float u = a.uniforms[slot];
    int pick = 0x7fffffff;
    if (n > 0) {
        // first unit whose final value passes the test holds the pick (the running sum never decreases)
        int ustar = 0x7fffffff;
        for (int u0 = 0; u0 < nun && ustar == 0x7fffffff; u0 += 64) {
            const int c = u0 + lane;
            const bool hit = c < nun && cp[c] / acc >= u;
            const unsigned long long m = __ballot(hit);
            if (m) ustar = u0 + (int)__ffsll((long long)m) - 1;
        }
        if (ustar != 0x7fffffff) {
            float run = ustar > 0 ? cp[ustar - 1] : 0.0f;
            const int i = ustar * 32 + lane;
            const float p = (lane < 32 && i < V) ? pk[i] : 0.0f;
            for (int j = 0; j < 32 && ustar * 32 + j < n; ++j) {
                run += __shfl(p, j, 64);
                if (run / acc >= u) { pick = ustar * 32 + j; break; }
            }
        }
    }
    if (lane == 0) {
        const int id = pick == 0x7fffffff ? 0 : idx[pick];
        if (a.next_ids) a.next_ids[r] = id;
        if (a.gen_out) a.gen_out[slot] = id;
        if (a.out_f32) a.out_f32[r] = (float)id;
        if (a.record && a.last_pos) a.last_pos[(long)r * a.last_ld + id] = topp_seq_len(a, r);     // the new token's index
    }
}

// the whole pipeline; `launch_fn(name, kernel, grid, block, args)` puts one kernel on the library stream
template <typename LaunchFn>
inline void topp_run(TopPArgs a, int rows, LaunchFn&& launch_fn) {
    launch_fn("topp_keys", topp_keys_kernel, dim3((unsigned)rows), dim3(1024), a);
    for (int pass = 0; pass < 4; ++pass) {
        a.shift = pass * 8;
        launch_fn("topp_hist", topp_hist_kernel, dim3((unsigned)a.nseg, (unsigned)rows), dim3(256), a);
        launch_fn("topp_scan", topp_scan_kernel, dim3((unsigned)rows), dim3(256), a);
        launch_fn("topp_scatter", topp_scatter_kernel, dim3((unsigned)a.nseg, (unsigned)rows), dim3(256), a);
        unsigned* tk = a.keysA; a.keysA = a.keysB; a.keysB = tk;
        int* ti = a.idxA; a.idxA = a.idxB; a.idxB = ti;
    }
    launch_fn("topp_pick", topp_pick_kernel, dim3((unsigned)rows), dim3(64), a);
}

}  // namespace tship
