// Measurement aid: what the decode step's launch structure costs on this machine with every kernel replaced by a pure
// streaming read of the same bytes.  A decode step is a chain of phases (projection, attention, projection, ...), each of
// which reads its weights or cache once and depends on the phase before it through a small activation tensor.  The probe
// runs such a chain three ways over real device memory and reports the time of each:
//   0: one kernel launch per phase (the structure the fused path uses);
//   1: one persistent kernel, one block per compute unit, phases separated by a grid-wide barrier (an agent-scope counter,
//      bounded polling);
//   2: the same with every wavefront requesting its first batch of the next phase before it arrives at the barrier;
//   4: one launch per phase, except that the phases marked in `fuse_with_next` share a launch with their successor: a
//      resident kernel (one block per compute unit) runs both with one grid-wide barrier in between, every wavefront
//      requesting its first batch of the second phase before it arrives at the barrier (half-layer fusion: the output
//      projection with the FFN up projection, the FFN down projection with the next QKV projection);
//   3: one launch per phase again, but every phase reads the same region from offset 0, so that after the first phases the
//      bytes come from the memory-side cache where they fit: what is left is the cost of the launch edges themselves, and
//      the distance to (0) is what prefetching the next phase's weights into that cache could gain at most.
// Every phase also reads `act_kib` KiB that all blocks share (the activations every column tile needs) and leaves one
// float per thread for the next phase to read from another block (the dependency).  No arithmetic beyond additions.
#include "tship_internal.h"

#include <vector>

namespace tship {

constexpr int PROBE_U = 8, PROBE_NT = 512, PROBE_NW = PROBE_NT / 64, PROBE_MAXP = 128;
struct ProbePhase { long off16; long chunks; int act_kib; };
struct ProbePlan { int n; ProbePhase p[PROBE_MAXP]; };

__device__ __forceinline__ void probe_load(const floatx4* __restrict__ src, long off16, long c, long c1, int lane, floatx4 (&v)[PROBE_U]) {
#pragma unroll
    for (int u = 0; u < PROBE_U; ++u) { const long cc = max(min(c + u, c1 - 1), 0l); v[u] = src[off16 + cc * 64 + lane]; }
}

__device__ __forceinline__ floatx4 probe_stream(const floatx4* __restrict__ src, const ProbePhase& ph, int nblocks, int blk, int lane, int w, floatx4 (&v)[PROBE_U], bool have) {
    floatx4 acc = {0, 0, 0, 0};
    const long per = (ph.chunks + nblocks - 1) / nblocks;
    const long c0 = blk * per, c1 = min(c0 + per, ph.chunks);
    long c = c0 + (long)w * PROBE_U;
    if (!have && c < c1) probe_load(src, ph.off16, c, c1, lane, v);
    while (c < c1) {
        floatx4 nv[PROBE_U];
        const long cn = c + (long)PROBE_NW * PROBE_U;
        const bool more = cn < c1;
        if (more) probe_load(src, ph.off16, cn, c1, lane, nv);
#pragma unroll
        for (int u = 0; u < PROBE_U; ++u) acc += v[u];
        if (more) {
#pragma unroll
            for (int u = 0; u < PROBE_U; ++u) v[u] = nv[u];
        }
        c = cn;
    }
    return acc;
}

__global__ __launch_bounds__(PROBE_NT) void probe_phase_kernel(const floatx4* __restrict__ src, ProbePhase ph, int p, const floatx4* __restrict__ act,
                                                                float* xw, const float* xr, float* sink) {
    const int t = threadIdx.x, lane = t & 63, w = t >> 6, blk = blockIdx.x, nb = gridDim.x;
    float carry = xr ? xr[(long)((blk + 37) % nb) * PROBE_NT + t] : 0.0f;
    floatx4 v[PROBE_U];
    floatx4 a0 = {0, 0, 0, 0};
    if (xr) for (int i = t; i < ph.act_kib * 64; i += PROBE_NT) a0 += act[(long)(p & 3) * 16384 + i];
    floatx4 acc = probe_stream(src, ph, nb, blk, lane, w, v, false) + a0;
    xw[(long)blk * PROBE_NT + t] = acc[0] + carry;
    if (acc[0] + acc[1] + acc[2] + acc[3] == 1234.5f) sink[0] = acc[0];
}

template <bool PREFETCH>
__global__ __launch_bounds__(PROBE_NT) void probe_persistent_kernel(const floatx4* __restrict__ src, ProbePlan plan, const floatx4* __restrict__ act, float* xbuf,
                                                                     unsigned* counter, int* err, float* sink, int spin_limit) {
    const int t = threadIdx.x, lane = t & 63, w = t >> 6, blk = blockIdx.x, nb = gridDim.x;
    floatx4 total = {0, 0, 0, 0};
    floatx4 v[PROBE_U];
    bool have = false;
    float carry = 0.0f;
    for (int p = 0; p < plan.n; ++p) {
        const ProbePhase ph = plan.p[p];
        if (p > 0) {
            const float* xb = xbuf + (long)((p - 1) & 1) * nb * PROBE_NT;
            carry += __hip_atomic_load(xb + (long)((blk + 37) % nb) * PROBE_NT + t, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            for (int i = t; i < ph.act_kib * 64; i += PROBE_NT) total += act[(long)(p & 3) * 16384 + i];
        }
        total += probe_stream(src, ph, nb, blk, lane, w, v, have);
        have = false;
        if (p + 1 < plan.n) {
            if (PREFETCH) {
                const ProbePhase pn = plan.p[p + 1];
                const long pern = (pn.chunks + nb - 1) / nb;
                const long n0 = blk * pern, n1 = min(n0 + pern, pn.chunks);
                if (n0 + (long)w * PROBE_U < n1) { probe_load(src, pn.off16, n0 + (long)w * PROBE_U, n1, lane, v); have = true; }
            }
            float* xb = xbuf + (long)(p & 1) * nb * PROBE_NT;
            __hip_atomic_store(xb + (long)blk * PROBE_NT + t, total[0] + carry, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");       // the phase's output has reached memory before the block arrives
            __syncthreads();
            if (t == 0) {
                __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                const unsigned target = (unsigned)(p + 1) * nb;
                int spins = 0;
                while (__hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target) {
                    __builtin_amdgcn_s_sleep(1);
                    if (++spins > spin_limit) { *err = 1; break; }      // bounded: every block leaves the loop and the kernel ends
                }
            }
            __syncthreads();
        }
    }
    if (total[0] + total[1] + total[2] + total[3] + carry == 1234.5f) sink[0] = total[0];
}

// two phases in one launch, one grid barrier between them (bounded polling); grid = one block per compute unit
__global__ __launch_bounds__(PROBE_NT) void probe_pair_kernel(const floatx4* __restrict__ src, ProbePhase pa, ProbePhase pb, int p, const floatx4* __restrict__ act,
                                                               float* xa, const float* xr, float* xb, unsigned* counter, int* err, float* sink, int spin_limit) {
    const int t = threadIdx.x, lane = t & 63, w = t >> 6, blk = blockIdx.x, nb = gridDim.x;
    float carry = xr ? xr[(long)((blk + 37) % nb) * PROBE_NT + t] : 0.0f;
    floatx4 v[PROBE_U];
    floatx4 a0 = {0, 0, 0, 0};
    if (xr) for (int i = t; i < pa.act_kib * 64; i += PROBE_NT) a0 += act[(long)(p & 3) * 16384 + i];
    floatx4 acc = probe_stream(src, pa, nb, blk, lane, w, v, false) + a0;
    // first batch of the second phase, requested before the barrier
    bool have = false;
    {
        const long pern = (pb.chunks + nb - 1) / nb;
        const long n0 = blk * pern, n1 = min(n0 + pern, pb.chunks);
        if (n0 + (long)w * PROBE_U < n1) { probe_load(src, pb.off16, n0 + (long)w * PROBE_U, n1, lane, v); have = true; }
    }
    __hip_atomic_store(xa + (long)blk * PROBE_NT + t, acc[0] + carry, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (t == 0) {
        __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        int spins = 0;
        while (__hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < (unsigned)nb) {
            __builtin_amdgcn_s_sleep(1);
            if (++spins > spin_limit) { *err = 1; break; }          // bounded: every block leaves the loop and the kernel ends
        }
    }
    __syncthreads();
    carry = __hip_atomic_load(xa + (long)((blk + 37) % nb) * PROBE_NT + t, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    floatx4 b0 = {0, 0, 0, 0};
    for (int i = t; i < pb.act_kib * 64; i += PROBE_NT) b0 += act[(long)((p + 1) & 3) * 16384 + i];
    floatx4 acc2 = probe_stream(src, pb, nb, blk, lane, w, v, have) + b0;
    xb[(long)blk * PROBE_NT + t] = acc2[0] + carry;
    if (acc[0] + acc2[0] + acc2[1] + acc2[2] + acc2[3] == 1234.5f) sink[0] = acc[0];
}

}  // namespace tship

using namespace tship;

extern "C" TSHIP_API int TSHip_StreamStructureProbe(int n_phases, const double* phase_bytes, const int* act_kib, const int* fuse_with_next, int repeats, float* ms_out /* [5] */) {
    TSHIP_BEGIN
    TSHIP_REQUIRE(phase_bytes && act_kib && ms_out, "TSHip_StreamStructureProbe: null argument");
    TSHIP_REQUIRE(n_phases >= 1 && n_phases <= PROBE_MAXP && repeats >= 1, "TSHip_StreamStructureProbe: between 1 and 128 phases");
    ensure_init();
    const int nb = n_compute_units();
    ProbePlan plan; plan.n = n_phases;
    long off = 0;
    for (int i = 0; i < n_phases; ++i) {
        TSHIP_REQUIRE(phase_bytes[i] >= 0 && act_kib[i] >= 0 && act_kib[i] <= 256, "TSHip_StreamStructureProbe: bad phase");
        const long chunks = (long)(phase_bytes[i] / 1024.0);
        plan.p[i] = ProbePhase{off * 64, chunks, act_kib[i]};
        off += chunks;
    }
    const size_t total = (size_t)std::max<long>(off, 1) * 1024;
    void *buf = nullptr, *act = nullptr, *xbuf = nullptr, *misc = nullptr;
    auto cleanup = [&]() { (void)hipStreamSynchronize(stream()); for (void* p : {buf, act, xbuf, misc}) if (p) (void)hipFree(p); };
    try {
        TSHIP_CHECK_HIP(hipMalloc(&buf, total));
        TSHIP_CHECK_HIP(hipMalloc(&act, 4 * 16384 * 16));
        TSHIP_CHECK_HIP(hipMalloc(&xbuf, 2l * nb * PROBE_NT * sizeof(float)));
        TSHIP_CHECK_HIP(hipMalloc(&misc, 4096));
        TSHIP_CHECK_HIP(hipMemsetAsync(buf, 0, total, stream()));
        TSHIP_CHECK_HIP(hipMemsetAsync(act, 0, 4 * 16384 * 16, stream()));
        TSHIP_CHECK_HIP(hipMemsetAsync(xbuf, 0, 2l * nb * PROBE_NT * sizeof(float), stream()));
        unsigned* counter = (unsigned*)misc; int* err = (int*)((char*)misc + 256); float* sink = (float*)((char*)misc + 512);
        float* xb = (float*)xbuf;
        hipEvent_t e0, e1;
        TSHIP_CHECK_HIP(hipEventCreate(&e0)); TSHIP_CHECK_HIP(hipEventCreate(&e1));
        for (int variant = 0; variant < 5; ++variant) {
            if (variant == 4 && !fuse_with_next) { ms_out[4] = 0.0f; continue; }
            float best = 1e30f;
            for (int it = 0; it < repeats; ++it) {
                TSHIP_CHECK_HIP(hipMemsetAsync(misc, 0, 4096, stream()));
                TSHIP_CHECK_HIP(hipEventRecord(e0, stream()));
                if (variant == 0 || variant == 3) {
                    for (int p = 0; p < plan.n; ++p) {
                        ProbePhase ph = plan.p[p];
                        if (variant == 3) ph.off16 = 0;
                        hipLaunchKernelGGL(probe_phase_kernel, dim3(nb), dim3(PROBE_NT), 0, stream(), (const floatx4*)buf, ph, p, (const floatx4*)act,
                                           xb + (long)(p & 1) * nb * PROBE_NT, p ? xb + (long)((p - 1) & 1) * nb * PROBE_NT : (const float*)nullptr, sink);
                    }
                } else if (variant == 4) {
                    unsigned* counters = (unsigned*)((char*)misc + 1024);          // one counter per fused launch
                    int slot = 0;
                    for (int p = 0; p < plan.n; ++p) {
                        float* xw = xb + (long)(p & 1) * nb * PROBE_NT;
                        const float* xr = p ? xb + (long)((p - 1) & 1) * nb * PROBE_NT : (const float*)nullptr;
                        if (fuse_with_next[p] && p + 1 < plan.n) {
                            hipLaunchKernelGGL(probe_pair_kernel, dim3(nb), dim3(PROBE_NT), 0, stream(), (const floatx4*)buf, plan.p[p], plan.p[p + 1], p, (const floatx4*)act,
                                               xw, xr, xb + (long)((p + 1) & 1) * nb * PROBE_NT, counters + slot, err, sink, 2000000);
                            ++slot; ++p;
                        } else {
                            hipLaunchKernelGGL(probe_phase_kernel, dim3(nb), dim3(PROBE_NT), 0, stream(), (const floatx4*)buf, plan.p[p], p, (const floatx4*)act, xw, xr, sink);
                        }
                    }
                } else if (variant == 1) {
                    hipLaunchKernelGGL(probe_persistent_kernel<false>, dim3(nb), dim3(PROBE_NT), 0, stream(), (const floatx4*)buf, plan, (const floatx4*)act, xb, counter, err, sink, 2000000);
                } else {
                    hipLaunchKernelGGL(probe_persistent_kernel<true>, dim3(nb), dim3(PROBE_NT), 0, stream(), (const floatx4*)buf, plan, (const floatx4*)act, xb, counter, err, sink, 2000000);
                }
                TSHIP_CHECK_HIP(hipGetLastError());
                TSHIP_CHECK_HIP(hipEventRecord(e1, stream()));
                TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));
                float ms = 0.0f;
                TSHIP_CHECK_HIP(hipEventElapsedTime(&ms, e0, e1));
                best = std::min(best, ms);
                int herr = 0;
                TSHIP_CHECK_HIP(hipMemcpy(&herr, err, sizeof(int), hipMemcpyDeviceToHost));
                TSHIP_REQUIRE(herr == 0, "TSHip_StreamStructureProbe: a grid barrier ran into its polling limit (are all compute units free?)");
            }
            ms_out[variant] = best;
        }
        (void)hipEventDestroy(e0); (void)hipEventDestroy(e1);
    } catch (...) { cleanup(); throw; }
    cleanup();
    TSHIP_END
}
