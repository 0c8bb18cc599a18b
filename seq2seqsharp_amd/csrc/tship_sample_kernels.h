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
// blocks); the running sum has the values of the reference's one-by-one fp32 additions (computed with block-wide scans
// in integer arithmetic, see topp_pick_scan_kernel), so for given probabilities the chosen index is the reference's,
// bit for bit.
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
    int scan_in_scatter;                   // the scatter kernel turns the digit counts into offsets itself (rows of up to 64 segments)
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

// Softmax statistics of a row, a row split over its nseg segments of 1024 elements so that the whole chip works on the
// rows: per-segment maxima, then per-segment sums of exp(x / T - row maximum).  They live in the first floats of the
// row's slice of `accp`, which the pick kernel only uses afterwards: maxima at [seg], sums at [nseg + seg].
// grid (nseg, rows), 256 threads, four elements per thread.
static __global__ __launch_bounds__(256) void topp_rowmax_kernel(TopPArgs a) {
    __shared__ float sred[4];
    const int seg = blockIdx.x, r = blockIdx.y, t = threadIdx.x;
    const float* row = a.in + (long)r * a.ld;
    float lm = -INFINITY;
#pragma unroll
    for (int it = 0; it < 4; ++it) {
        const int i = seg * TOPP_SEG + it * 256 + t;
        if (i < a.V) lm = fmaxf(lm, row[i] / a.temperature);
    }
    const float m = block_max_256(lm, sred);
    if (t == 0) a.accp[(long)r * a.Vs + seg] = m;
}

__device__ __forceinline__ float topp_row_max(const TopPArgs& a, int r) {
    const float* sm = a.accp + (long)r * a.Vs;
    float mx = sm[0];
    for (int s2 = 1; s2 < a.nseg; ++s2) mx = fmaxf(mx, sm[s2]);
    return mx;
}

static __global__ __launch_bounds__(256) void topp_rowsum_kernel(TopPArgs a) {
    __shared__ float sred[4];
    const int seg = blockIdx.x, r = blockIdx.y, t = threadIdx.x;
    const float* row = a.in + (long)r * a.ld;
    const float mx = topp_row_max(a, r);
    float ls = 0.0f;
#pragma unroll
    for (int it = 0; it < 4; ++it) {
        const int i = seg * TOPP_SEG + it * 256 + t;
        if (i < a.V) ls += expf(row[i] / a.temperature - mx);
    }
    ls = wave_sum(ls);
    if ((t & 63) == 0) sred[t >> 6] = ls;
    __syncthreads();
    if (t == 0) a.accp[(long)r * a.Vs + a.nseg + seg] = ((sred[0] + sred[1]) + sred[2]) + sred[3];
}

// probabilities (TensorApplyCPU.Softmax, TensorApplyCPU.cs:1230-1268) written as sort keys, and the digit counts of the
// first sort pass: grid (nseg, rows), 256 threads.  The row's sum is the sum of the segment sums in segment order.
static __global__ __launch_bounds__(256) void topp_keys_kernel(TopPArgs a) {
    __shared__ unsigned s_key[TOPP_SEG];
    __shared__ int s_hist[256];
    const int seg = blockIdx.x, r = blockIdx.y, t = threadIdx.x, V = a.V;
    const int i0 = seg * TOPP_SEG;
    const float* row = a.in + (long)r * a.ld;
    unsigned* kA = a.keysA + (long)r * a.Vs;
    int* iA = a.idxA + (long)r * a.Vs;
    float sum = 1.0f, mx = 0.0f;
    if (a.in_is_logits) {
        mx = topp_row_max(a, r);
        const float* ss = a.accp + (long)r * a.Vs + a.nseg;
        sum = ss[0];
        for (int s2 = 1; s2 < a.nseg; ++s2) sum += ss[s2];
    }
    // Repeat penalty: few tokens of the vocabulary occur in the sequence, but almost every wavefront holds one of them, and
    // the double-precision pow would be paid by all 64 lanes.  So the pass over the segment only notes those tokens
    // (index and probability) in an LDS list, and the list is worked off densely afterwards.
    __shared__ int s_didx[TOPP_SEG];
    __shared__ float s_dp[TOPP_SEG];
    __shared__ int s_dn;
    const bool decay = a.last_pos && a.repeat_penalty != 0.0f;
    const int len = decay ? topp_seq_len(a, r) : 0;
    const int* last = decay ? a.last_pos + (long)r * a.last_ld : nullptr;
    auto decayed = [&](float p, int lp) {
        // float division, double pow, one rounding to float, one fp32 multiply (ComputeGraphTensor.cs:2341-2342)
        const float ratio = (float)(len - lp) / (float)len;
        const float rp = (float)pow((double)ratio, (double)a.repeat_penalty);
        return p * rp;          // (a product that underflows to 0 stays a candidate of weight 0 there; it can never be picked)
    };
    // p > 0: positive floats order like their bit patterns; descending order = ascending ~bits.
    // p <= 0 is dropped by the reference: give it the largest key so that it sorts behind every candidate.
    auto key_of = [&](float p, int i) { return (p > 0.0f && !(a.blocked && a.blocked[i])) ? ~__float_as_uint(p) : 0xffffffffu; };
    if (t == 0) s_dn = 0;
    s_hist[t] = 0;
    __syncthreads();
#pragma unroll
    for (int it = 0; it < 4; ++it) {
        const int e = it * 256 + t, i = i0 + e;
        if (i >= V) continue;
        const float p = a.in_is_logits ? expf(row[i] / a.temperature - mx) / sum : row[i];
        if (decay && p > 0.0f) {
            const int lp = last[i];
            if (lp >= 0) { const int slot = atomicAdd(&s_dn, 1); s_didx[slot] = e; s_dp[slot] = p; }      // (at most TOPP_SEG entries)
        }
        s_key[e] = key_of(p, i);
    }
    __syncthreads();
    if (decay) {
        const int nd = s_dn;
        for (int k = t; k < nd; k += 256) {
            const int e = s_didx[k], i = i0 + e;
            s_key[e] = key_of(decayed(s_dp[k], last[i]), i);
        }
        __syncthreads();
    }
#pragma unroll
    for (int it = 0; it < 4; ++it) {
        const int e = it * 256 + t, i = i0 + e;
        if (i >= V) continue;
        const unsigned k = s_key[e];
        kA[i] = k; iA[i] = i;
        atomicAdd(&s_hist[k & 255u], 1);
    }
    __syncthreads();
    a.hist[((long)r * a.nseg + seg) * 256 + t] = s_hist[t];
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
        int run;
        if (a.scan_in_scatter) {
            // offset of (segment, digit t) in (digit major, segment minor) order from the row's raw counts: the digit's counts in
            // the segments before this one, plus the totals of all smaller digits (what topp_scan_kernel leaves in `hist`;
            // every block of the row repeats the sums, which costs less than a launch of its own between histogram and scatter)
            __shared__ int tot[256];
            const int* h = a.hist + (long)r * a.nseg * 256;
            int before = 0, total = 0;
            for (int s0 = 0; s0 < a.nseg; s0 += 8) {
                int v[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) v[u] = s0 + u < a.nseg ? h[(s0 + u) * 256 + t] : 0;
#pragma unroll
                for (int u = 0; u < 8; ++u) { total += v[u]; if (s0 + u < seg) before += v[u]; }
            }
            tot[t] = total;
            __syncthreads();
            if (t < 64) {       // one wavefront: 4 digits per lane, then a shuffle scan over the lane sums
                const int v0 = tot[4 * t], v1 = tot[4 * t + 1], v2 = tot[4 * t + 2], v3 = tot[4 * t + 3];
                const int mine = v0 + v1 + v2 + v3;
                int inc = mine;
#pragma unroll
                for (int o = 1; o < 64; o <<= 1) { const int n = __shfl_up(inc, o, 64); if (t >= o) inc += n; }
                const int base = inc - mine;
                tot[4 * t] = base; tot[4 * t + 1] = base + v0; tot[4 * t + 2] = base + v0 + v1; tot[4 * t + 3] = base + v0 + v1 + v2;
            }
            __syncthreads();
            run = tot[t] + before;
        } else {
            run = a.hist[((long)r * a.nseg + seg) * 256 + t];
        }
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

// ------------------------------------------------------------------------------------------------
// Running sum and pick, evaluated in parallel but with the values of the sequential fp32 sum, bit for bit.
//
// The reference adds the sorted probabilities one by one in fp32: acc_k = fl(acc_{k-1} + p_k).  While acc stays inside
// one binade [2^e, 2^(e+1)) it is an integer multiple A of u = 2^(e-23), and (p_k <= acc, so p_k's exponent is not
// larger) the rounded sum is A + d_k with d_k = floor(p_k / u) + 1 if the fraction of p_k / u is above 1/2, + 0 if below,
// and on an exact tie whatever makes A + d_k even (round to nearest even).  floor and fraction come from shifting p_k's
// 24-bit significand, so d_k is integer arithmetic; a tie makes d_k depend on the parity of the sum before it, and that
// parity runs through the elements as a composition of maps "xor with a bit" / "constant 0", which is associative.  Two
// block-wide scans (parity maps, then integers) therefore give every acc_k of a tile at once.  The element at which
// the sum leaves the binade is added in floating point by itself, and the next tile starts behind it with the new u.
// The first PICK_HEAD elements are added one by one by a single thread: the sum changes binade after 2, 4, 8 ...
// elements of a flat distribution, and a peaked one (a trained model) reaches top_p within them, so the scans never start.
// grid (rows), 512 threads; eight consecutive elements per thread and tile (256, 512 and 1024 threads measured the same
// within 15 %: the kernel is bound by its instruction count on one CU, about 60 per element and pass).
// ------------------------------------------------------------------------------------------------
constexpr int PICK_E = 8, PICK_THREADS = 512, PICK_WAVES = PICK_THREADS / 64, PICK_TILE = PICK_E * PICK_THREADS;
constexpr int PICK_HEAD = 512;                          // elements added one by one before the scans start
constexpr unsigned PICK_CAP = 1u << 25;                  // sums saturate here: anything >= 2^24 has left the binade

__device__ __forceinline__ unsigned pick_sat_add(unsigned a, unsigned b) { const unsigned s = a + b; return s > PICK_CAP ? PICK_CAP : s; }
// parity maps in two bits: bit 1 = constant, bit 0 = the constant or the xor mask; `then(prev, cur)` = cur after prev
__device__ __forceinline__ unsigned pick_map_then(unsigned prev, unsigned cur) { return (cur & 2u) ? cur : ((prev & 2u) | ((prev ^ cur) & 1u)); }
__device__ __forceinline__ unsigned pick_map_apply(unsigned map, unsigned parity) { return (map & 2u) ? (map & 1u) : ((parity ^ map) & 1u); }

// inclusive scan of saturating sums over the 64 lanes with data-parallel-primitive moves (no LDS): shifts by 1, 2, 4, 8
// inside rows of 16 lanes, then the last lane of row 0 / 2 into rows 1 / 3 and of row 1 into rows 2 and 3
__device__ __forceinline__ unsigned pick_wave_scan(unsigned x) {
    x = pick_sat_add(x, (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, 0x111, 0xf, 0xf, false));
    x = pick_sat_add(x, (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, 0x112, 0xf, 0xf, false));
    x = pick_sat_add(x, (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, 0x114, 0xf, 0xf, false));
    x = pick_sat_add(x, (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, 0x118, 0xf, 0xf, false));
    x = pick_sat_add(x, (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, 0x142, 0xa, 0xf, false));
    x = pick_sat_add(x, (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, 0x143, 0xc, 0xf, false));
    return x;
}
// parity maps of the lanes below `lane`, composed, from two ballots (which lanes are constant, the lanes' low bits):
// the last constant lane below fixes the value, the xor bits above it flip it
__device__ __forceinline__ unsigned pick_map_below(unsigned long long isc, unsigned long long bit, int lane) {
    const unsigned long long lower = (1ull << lane) - 1ull;
    const unsigned long long c = isc & lower;
    if (c == 0ull) return (unsigned)__popcll(bit & lower) & 1u;
    const int q = 63 - __clzll((long long)c);
    const unsigned long long above = lower & ~((2ull << q) - 1ull);
    return 2u | ((((unsigned)(bit >> q)) ^ (unsigned)__popcll(bit & above)) & 1u);
}

// block barrier that orders LDS traffic only (outstanding global stores are not waited for)
__device__ __forceinline__ void pick_lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// (the chosen token is returned to every thread of the block)
__device__ __forceinline__ int topp_pick_scan_row(const TopPArgs& a) {
    __shared__ unsigned s_wmap[PICK_WAVES], s_wsum[PICK_WAVES];
    __shared__ int s_id;
    __shared__ int s_event[PICK_WAVES];
    __shared__ float s_acc;
    __shared__ int s_j0, s_n, s_state, s_pick[PICK_WAVES];
    __shared__ float s_head[PICK_HEAD];                     // s_state: 0 = go on in this tile, 1 = next tile, 2 = finished
    const int r = blockIdx.x, t = threadIdx.x, lane = t & 63, w = t >> 6, V = a.V;
    const unsigned* pk = a.keysA + (long)r * a.Vs;                   // sorted probabilities as bit patterns, 0 = not a candidate
    const int* idx = a.idxA + (long)r * a.Vs;
    float* accp = a.accp + (long)r * a.Vs;                           // accp[k]: running sum after element k
    // a tile's bit patterns are fetched once (two 16-byte loads per thread: Vs is a multiple of 64 elements), the next
    // tile's while this one is worked on
    unsigned bits[PICK_E], nbits[PICK_E];
    auto tile_load = [&](int kb, unsigned (&dst)[PICK_E]) {
        const int k = kb + t * PICK_E;
        uint4 lo = uint4{0u, 0u, 0u, 0u}, hi = lo;
        if (k < a.Vs) { lo = *(const uint4*)(pk + k); hi = *(const uint4*)(pk + k + 4); }     // k + 7 < Vs
        dst[0] = lo.x; dst[1] = lo.y; dst[2] = lo.z; dst[3] = lo.w; dst[4] = hi.x; dst[5] = hi.y; dst[6] = hi.z; dst[7] = hi.w;
#pragma unroll
        for (int i = 0; i < PICK_E; ++i) if (k + i >= V) dst[i] = 0u;                         // padding is not a candidate
    };
    tile_load(0, bits);
    // head of the row, one by one (starting from acc = 0 as the reference does).  Wavefront 0 holds these elements (lane L:
    // 8 L .. 8 L + 7); they are broadcast lane by lane into scalar registers, so one element costs a read-lane and one add.
    if (w == 0) {
        float acc = 0.0f; int k = 0; bool stop = false;
        for (int L = 0; L < PICK_HEAD / PICK_E && !stop; ++L) {
            float pv[PICK_E];
#pragma unroll
            for (int i = 0; i < PICK_E; ++i) pv[i] = __uint_as_float((unsigned)__builtin_amdgcn_readlane((int)bits[i], L));
#pragma unroll
            for (int i = 0; i < PICK_E; ++i) {
                if (stop) break;
                if (!(pv[i] > 0.0f)) { stop = true; break; }         // no more candidates (padding behind V is 0 as well)
                acc += pv[i];
                if (lane == 0) s_head[k] = acc;
                ++k;
                if (acc >= a.top_p) stop = true;
            }
        }
        if (lane == 0) { s_acc = acc; s_n = k; s_j0 = k; s_state = stop ? 2 : 0; }
    }
    __syncthreads();
    for (int k = t; k < s_n && k < PICK_HEAD; k += PICK_THREADS) accp[k] = s_head[k];
    for (int kb = 0; s_state != 2; kb += PICK_TILE) {
        if (kb + PICK_TILE < V) tile_load(kb + PICK_TILE, nbits);
        // work through this tile; every pass ends at an event: the sum leaves its binade (another pass), reaches top_p,
        // runs out of candidates, or the tile ends
        for (;;) {
            const int j0 = s_j0;                                     // elements of the tile before j0 are done
            const float acc0 = s_acc;
            const unsigned abits = __float_as_uint(acc0);
            const int aexp = (int)(abits >> 23);                     // biased; 0 = subnormal
            pick_lds_barrier();                                         // everyone has read the state
            if (j0 >= PICK_TILE) { if (t == 0) { s_state = 1; } pick_lds_barrier(); break; }
            if (aexp <= 23) {
                // a running sum below 2^-103, where 2^(e-23) is not a normal float (never after a softmax): one plain step
                if (t == 0) {
                    const int k = kb + j0;
                    const float p = k < V ? __uint_as_float(pk[k]) : 0.0f;
                    if (p > 0.0f) { const float v = acc0 + p; accp[k] = v; s_acc = v; s_j0 = j0 + 1; s_n = k + 1; if (v >= a.top_p) s_state = 2; }
                    else s_state = 2;
                }
                pick_lds_barrier();
                if (s_state == 2) break;
                continue;
            }
            const unsigned A0 = (abits & 0x7fffffu) | 0x800000u;
            unsigned dfl[PICK_E], cls[PICK_E];                       // cls: 0 plain (d = dfl), 1 tie, 2 not a candidate, 3 already done
            unsigned map = 0u;                                       // identity
#pragma unroll
            for (int i = 0; i < PICK_E; ++i) {
                const unsigned b = bits[i];
                dfl[i] = 0u;
                if (t * PICK_E + i < j0) { cls[i] = 3u; continue; }
                if (b == 0u) { cls[i] = 2u; continue; }              // (sorted: everything behind it is 0 as well)
                const int pexp = (int)(b >> 23);
                const unsigned m = pexp ? ((b & 0x7fffffu) | 0x800000u) : (b & 0x7fffffu);
                const int sh = aexp - (pexp ? pexp : 1);             // >= 0: p <= acc
                if (sh < 0) { dfl[i] = PICK_CAP; cls[i] = 0u; continue; }   // not sorted (NaN in the input): handled as leaving the binade
                // m / 2^sh as 32.32 fixed point: integer part and the fraction, which the shift leaves exact (sh <= 32)
                const unsigned long long x = sh <= 32 ? (((unsigned long long)m << 32) >> sh) : 0ull;      // sh > 32: below 1/2
                const unsigned fl = (unsigned)(x >> 32), frac = (unsigned)x;
                const bool gt = frac > 0x80000000u, tie = frac == 0x80000000u;
                dfl[i] = fl + (gt ? 1u : 0u); cls[i] = tie ? 1u : 0u;
                map = pick_map_then(map, tie ? 2u : (dfl[i] & 1u));
            }
            // exclusive scan of the parity maps over the block
            const unsigned long long b_isc = __ballot((map & 2u) != 0u), b_bit = __ballot((map & 1u) != 0u);
            if (lane == 63) s_wmap[w] = pick_map_then(pick_map_below(b_isc, b_bit, 63), map);        // the whole wavefront
            pick_lds_barrier();
            unsigned before = 0u;                                    // map of everything ahead of this thread
            for (int i = 0; i < w; ++i) before = pick_map_then(before, s_wmap[i]);
            before = pick_map_then(before, pick_map_below(b_isc, b_bit, lane));
            unsigned parity = pick_map_apply(before, A0 & 1u);
            // increments with the ties resolved, local prefix
            unsigned loc[PICK_E], run = 0u;
#pragma unroll
            for (int i = 0; i < PICK_E; ++i) {
                unsigned d = dfl[i];
                if (cls[i] == 1u) d += (parity ^ d) & 1u;            // make the sum even
                if (cls[i] >= 2u) d = 0u;
                parity = (parity ^ d) & 1u;
                run = pick_sat_add(run, d > PICK_CAP ? PICK_CAP : d);
                loc[i] = run;
            }
            const unsigned sinc = pick_wave_scan(run);              // inclusive over the wavefront
            if (lane == 63) s_wsum[w] = sinc;
            pick_lds_barrier();
            unsigned base = A0;
            for (int i = 0; i < w; ++i) base = pick_sat_add(base, s_wsum[i]);
            { const unsigned prev = __shfl_up(sinc, 1, 64); if (lane > 0) base = pick_sat_add(base, prev); }
            // values, and the first event: 4 j + type, type 0 = leaves the binade, 1 = reaches top_p, 2 = no more candidates
            // (val of an element at which the sum leaves the binade: the floating-point sum of the value before it and the
            // element; it is only used if that element turns out to be the first event)
            float val[PICK_E];
            int event = 0x7fffffff;
            const float scale = __uint_as_float((unsigned)(aexp - 23) << 23);      // 2^(e - 23) with e = aexp - 127: biased exponent aexp - 23 >= 1
            unsigned Aprev = base;
#pragma unroll
            for (int i = 0; i < PICK_E; ++i) {
                const int j = t * PICK_E + i;
                const unsigned A = pick_sat_add(base, loc[i]);
                val[i] = 0.0f;
                int ev = 0x7fffffff;
                if (cls[i] == 3u) ev = 0x7fffffff;
                else if (cls[i] == 2u) ev = 4 * j + 2;
                else if (A >= (1u << 24)) { ev = 4 * j + 0; val[i] = (float)Aprev * scale + __uint_as_float(bits[i]); }
                else { val[i] = (float)A * scale; if (val[i] >= a.top_p) ev = 4 * j + 1; }
                if (ev < event) event = ev;
                Aprev = A;
            }
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) { const int other = __shfl_xor(event, o, 64); if (other < event) event = other; }
            if (lane == 0) s_event[w] = event;
            pick_lds_barrier();
            event = s_event[0];
#pragma unroll
            for (int i = 1; i < PICK_WAVES; ++i) event = min(event, s_event[i]);
            const int jstop = event == 0x7fffffff ? PICK_TILE : event >> 2, type = event == 0x7fffffff ? -1 : (event & 3);
            // elements ahead of the event are final; so is an element that reaches top_p or at which the sum leaves its
            // binade (one floating-point addition, done above)
            const int jkeep = (type == 1 || type == 0) ? jstop + 1 : jstop;
#pragma unroll
            for (int i = 0; i < PICK_E; ++i) {
                const int j = t * PICK_E + i;
                if (j >= j0 && j < jkeep) { accp[kb + j] = val[i]; if (j == jkeep - 1) s_acc = val[i]; }      // the last final value is the running sum
            }
            pick_lds_barrier();              // (the stores to accp are not waited for here: they are read after the loop)
            if (t == 0) {
                if (jkeep > j0) s_n = kb + jkeep;
                if (type == -1) { s_j0 = PICK_TILE; }
                else if (type == 1 || type == 2) { s_state = 2; }
                else { s_j0 = jstop + 1; if (s_acc >= a.top_p) s_state = 2; }
            }
            pick_lds_barrier();
            if (s_state == 2) break;
        }
        if (s_state == 2) break;
        // next tile
        pick_lds_barrier();
        if (t == 0) { s_state = kb + PICK_TILE < V ? 0 : 2; s_j0 = 0; }
#pragma unroll
        for (int i = 0; i < PICK_E; ++i) bits[i] = nbits[i];
        pick_lds_barrier();
    }
    __threadfence_block();
    __syncthreads();
    const int n = s_n;
    const float acc = s_acc;
    const long slot = (a.d_step ? (long)*a.d_step * gridDim.x : 0) + r;
    const float u = a.uniforms[slot];
    // first k < n with accp[k] / acc >= u.  The running sum never decreases, so the test is monotone in k: the last
    // elements of 512 equal segments locate the segment, its (at most 512) elements the index: two loads per thread.
    auto block_min = [&](int v) {
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) { const int other = __shfl_xor(v, o, 64); if (other < v) v = other; }
        __syncthreads();
        if (lane == 0) s_pick[w] = v;
        __syncthreads();
        int m = s_pick[0];
#pragma unroll
        for (int i = 1; i < PICK_WAVES; ++i) m = min(m, s_pick[i]);
        return m;
    };
    int pick = 0x7fffffff;
    if (n > 0) {
        const int seg = (n + PICK_THREADS - 1) / PICK_THREADS;           // <= 512 = PICK_THREADS: at most 262144 entries (checked by the callers)
        const int last = min(n, (t + 1) * seg) - 1;                      // last element of segment t (empty segments repeat n - 1)
        const int hit_seg = block_min((t * seg < n && accp[last] / acc >= u) ? t : 0x7fffffff);
        if (hit_seg != 0x7fffffff) {
            const int k = hit_seg * seg + t;
            pick = block_min((t < seg && k < n && accp[k] / acc >= u) ? k : 0x7fffffff);
        }
    }
    if (t == 0) {
        const int id = pick == 0x7fffffff ? 0 : idx[pick];
        if (a.next_ids) a.next_ids[r] = id;
        if (a.gen_out) a.gen_out[slot] = id;
        if (a.out_f32) a.out_f32[r] = (float)id;
        if (a.record && a.last_pos) a.last_pos[(long)r * a.last_ld + id] = topp_seq_len(a, r);     // the new token's index
        s_id = id;
    }
    __syncthreads();
    return s_id;
}
static __global__ __launch_bounds__(PICK_THREADS) void topp_pick_scan_kernel(TopPArgs a) { topp_pick_scan_row(a); }

// the whole pipeline; `launch_fn(name, kernel, grid, block, args)` puts one kernel on the library stream
// with_pick = false: everything but the last kernel; returns the arguments that kernel takes (the caller launches a pick
// kernel of its own, see topp_pick_embed_kernel)
template <typename LaunchFn>
inline TopPArgs topp_run(TopPArgs a, int rows, LaunchFn&& launch_fn, bool with_pick = true) {
    const dim3 segs((unsigned)a.nseg, (unsigned)rows);
    if (a.in_is_logits) {
        launch_fn("topp_rowmax", topp_rowmax_kernel, segs, dim3(256), a);
        launch_fn("topp_rowsum", topp_rowsum_kernel, segs, dim3(256), a);
    }
    a.scan_in_scatter = a.nseg <= 64 ? 1 : 0;      // (beyond that every block of a row would re-read too many counts)
    launch_fn("topp_keys", topp_keys_kernel, segs, dim3(256), a);          // also the digit counts of pass 0
    for (int pass = 0; pass < 4; ++pass) {
        a.shift = pass * 8;
        if (pass > 0) launch_fn("topp_hist", topp_hist_kernel, dim3((unsigned)a.nseg, (unsigned)rows), dim3(256), a);
        if (!a.scan_in_scatter) launch_fn("topp_scan", topp_scan_kernel, dim3((unsigned)rows), dim3(256), a);
        launch_fn("topp_scatter", topp_scatter_kernel, dim3((unsigned)a.nseg, (unsigned)rows), dim3(256), a);
        unsigned* tk = a.keysA; a.keysA = a.keysB; a.keysB = tk;
        int* ti = a.idxA; a.idxA = a.idxB; a.idxB = ti;
    }
    if (with_pick) launch_fn("topp_pick", topp_pick_scan_kernel, dim3((unsigned)rows), dim3(PICK_THREADS), a);
    return a;
}

}  // namespace tship
