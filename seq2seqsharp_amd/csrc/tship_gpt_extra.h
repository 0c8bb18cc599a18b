// Host side of the MoE feed-forward and of token sampling for the fused GPTDecoder path.
// Included by tship_gpt.hip after the model object is defined.
#pragma once

namespace tship {

struct MoeLayout {
    size_t xn32, probs, top_val, top_idx, counts, lists, slot, xg, mid, y, zero, total;
    long ld4h, ldy;
};

// cap: rows the workspace is laid out for (the padded batch for decode steps, the padded row count of a prefill)
static MoeLayout moe_layout(TSHipGpt* m, long cap) {
    auto& c = m->c;
    MoeLayout o; size_t at = 0;
    auto take = [&](size_t bytes) { size_t r = at; at += round_up((long)bytes, 256); return r; };
    const long h = c.hidden, E = c.n_experts, k = c.experts_per_token, Bp = cap;
    o.ld4h = round_up(4 * h, 16); o.ldy = round_up(h, 32);
    o.xn32 = take(Bp * h * 4); o.probs = take(Bp * E * 4); o.top_val = take(Bp * k * 4); o.top_idx = take(Bp * k * 4);
    o.counts = take(E * 4); o.lists = take(E * Bp * 4); o.slot = take(Bp * k * 4);
    o.xg = take(E * Bp * m->ldh * m->esz());
    o.mid = take(E * Bp * o.ld4h * m->esz());
    o.y = take(E * Bp * o.ldy * 4);
    o.zero = take(std::max<long>(4 * h, 64) * 4);
    o.total = at;
    return o;
}

static void moe_alloc(TSHipGpt* m) {
    TSHIP_REQUIRE(m->c.hidden <= 4096, "TSHip_GptCreate: MoE layers support hidden up to 4096");
    m->moe_ws.alloc(moe_layout(m, m->Bpad).total);
    // the experts' row counters start at zero and every layer's combine kernel leaves them so (the fp16 router adds to them)
    TSHIP_CHECK_HIP(hipMemsetAsync(m->moe_ws.p, 0, m->moe_ws.bytes, stream()));
}

static void moe_get_routing(TSHipGpt* m, int layer, float* top_idx, float* top_val, float* probs) {
    LayerW& L = *m->L[layer];
    const int B = m->cur_batch, k = m->c.experts_per_token, E = m->c.n_experts;
    TSHIP_REQUIRE(L.route.p, "TSHip_GptGetMoeRouting: call TSHip_GptFinalize first");
    TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));
    const float* base = L.route.as<float>();
    if (probs) TSHIP_CHECK_HIP(hipMemcpy(probs, base, (size_t)B * E * 4, hipMemcpyDeviceToHost));
    if (top_val) TSHIP_CHECK_HIP(hipMemcpy(top_val, base + (size_t)m->Bpad * E, (size_t)B * k * 4, hipMemcpyDeviceToHost));
    if (top_idx) TSHIP_CHECK_HIP(hipMemcpy(top_idx, base + (size_t)m->Bpad * (E + k), (size_t)B * k * 4, hipMemcpyDeviceToHost));
}

// `pre` carries the pending attention output (split-K partials + bias) and the LayerNorm parameters
// batched (prefill, any number of rows): the workspace is m->pw_moe laid out for `cap` rows, the lists come from the
// many-row kernel, the host reads the experts' row counts (the reference builds its lists on the host as well,
// MoEFeedForward.cs:92-105) and every expert with rows runs the prefill GEMMs on its gathered rows
// next: when given, the norm kernel that follows adds the experts' outputs itself (no separate combine launch)
// Prefills of fp16 models with 512 rows or more never read the counts back: the router writes the normalised rows as fp16,
// one launch per projection covers every expert's row tiles packed one behind the other (found on the device from the
// counts), and the up projection reads its rows through the token lists.
static void run_moe_ffn_impl(TSHipGpt* m, LayerW& L, int rows, const ResidNormArgs& pre, bool batched, long cap, const int* last_rows, int n_last,
                             const ResidNormArgs* next = nullptr) {
    auto& c = m->c;
    MoeLayout o = moe_layout(m, cap);
    char* base = (char*)(batched ? m->pw_moe.p : m->moe_ws.p);
    TSHIP_REQUIRE(rows <= cap && o.total <= (batched ? m->pw_moe.bytes : m->moe_ws.bytes), "internal: MoE workspace too small");
    const int h = c.hidden, E = c.n_experts, k = c.experts_per_token; const long Bp = cap;
    // decode steps write the routing straight into the layer's own buffers (TSHip_GptGetMoeRouting reads them); a prefill
    // routes all rows in the workspace and copies every sequence's last position there afterwards
    float* lroute = L.route.as<float>();
    TSHIP_REQUIRE(lroute && (size_t)m->Bpad * (E + 2 * k) * sizeof(float) <= L.route.bytes, "internal: routing buffers missing (TSHip_GptFinalize allocates them)");
    float* xn32 = (float*)(base + o.xn32); float* probs = batched ? (float*)(base + o.probs) : lroute;
    float* top_val = batched ? (float*)(base + o.top_val) : lroute + (size_t)m->Bpad * E;
    float* top_idx = batched ? (float*)(base + o.top_idx) : lroute + (size_t)m->Bpad * (E + k);
    int* counts = (int*)(base + o.counts); int* lists = (int*)(base + o.lists); int* slot = (int*)(base + o.slot);
    float* y = (float*)(base + o.y); float* zero = (float*)(base + o.zero);

    MoeRouterArgs r; std::memset(&r, 0, sizeof(r));
    r.x = pre.x; r.ldx = pre.ldx; r.h = h;
    r.part = pre.part; r.KS = pre.KS; r.split_stride = pre.split_stride; r.ld_part = pre.ld_part; r.bias = pre.bias;
    r.gamma = pre.gamma; r.beta = pre.beta; r.eps = pre.eps;
    r.router = L.router.as<float>(); r.router_b = L.router_b.as<float>(); r.E = E; r.k = k;
    r.xn32 = xn32; r.probs = probs; r.top_val = top_val; r.top_idx = top_idx;
    r.router_lds = ((long)E * h <= 16384) ? 1 : 0;
    const long xg_stride = (long)Bp * m->ldh, mid_stride = (long)Bp * o.ld4h, y_stride = (long)Bp * o.ldy;
    // fp16 decode steps: the router kernel also takes the row's place in its experts' batches and writes the row there
    const bool fused_route = m->f16 && h % 4 == 0 && !batched && k <= 64;
    if (fused_route) { r.xg16 = (half_t*)(base + o.xg); r.xg_estride = xg_stride; r.packed_kt = (int)(m->ldh / 16); r.counts = counts; r.slot = slot; r.max_rows = (int)Bp; }
    const bool packed = batched && m->f16 && h % 4 == 0 && rows >= 512 && big_gemm_batched_ok(*L.e1[0], rows) && big_gemm_batched_ok(*L.e2[0], rows) &&
                        L.wtab1.p && L.wtab2.p && !g_hooks.no_moe_batch;
    if (packed) { r.xn16 = (half_t*)(base + o.xg); r.ld_xn16 = m->ldh; }       // (the gathered rows' area holds them: E * cap rows are reserved)
    const unsigned router_shm = (unsigned)((2L * h + (r.router_lds ? (long)E * h : 0)) * sizeof(float));
    if (m->f16 && h % 4 == 0) {      // tree-order sums: an fp16 model's routing input is not the reference's to the last bit anyway
        if (h <= 1024) launch(m, "moe_router", moe_router_fast_kernel<1>, dim3(rows), dim3(256), r);
        else if (h <= 2048) launch(m, "moe_router", moe_router_fast_kernel<2>, dim3(rows), dim3(256), r);
        else launch(m, "moe_router", moe_router_fast_kernel<4>, dim3(rows), dim3(256), r);
    } else launch_shm(m, "moe_router", moe_router_kernel, dim3(rows), dim3(256), router_shm, r);
    // decode-sized batches: the gather kernel builds the lists itself (one launch less)
    const bool fused_lists = !batched && !fused_route && (long)rows * k <= 1024;
    if (batched) launch(m, "moe_lists", moe_lists_big_kernel, dim3(E), dim3(1024), (const float*)top_idx, rows, k, (int)Bp, counts, lists, slot);
    else if (!fused_lists && !fused_route) launch_shm(m, "moe_lists", moe_lists_kernel, dim3(1), dim3(64), (unsigned)(rows * k * sizeof(int)), (const float*)top_idx, rows, k, E, (int)Bp, counts, lists, slot);
    std::vector<int> n_e(E, rows);
    if (packed) {
        half_t* xn16 = (half_t*)(base + o.xg); half_t* mid = (half_t*)(base + o.mid);
        const int rt_bound = (int)((long)rows * k / 256 + E);      // >= the sum over the experts of ceil(count / 256)
        BigArgs e1; std::memset(&e1, 0, sizeof(e1));
        e1.bias = zero; e1.out16 = mid; e1.ld16 = (int)o.ld4h; e1.act = c.act; e1.gated = 0; e1.n_valid = 4 * h;
        e1.Wtab = (const half_t* const*)L.wtab1.p; e1.rows_tab = counts; e1.x_estride = 0; e1.out16_estride = mid_stride;
        e1.row_idx = lists; e1.idx_estride = Bp; e1.packed_problems = E; e1.packed_rt = rt_bound;
        run_big_gemm(m, "moe_gemm1", *L.e1[0], xn16, m->ldh, (long)rt_bound * 256, BEPI_ACT16, e1, E);
        BigArgs e2; std::memset(&e2, 0, sizeof(e2));
        e2.bias = zero; e2.out = y; e2.ld_out = (int)o.ldy; e2.n_valid = h;
        e2.Wtab = (const half_t* const*)L.wtab2.p; e2.rows_tab = counts; e2.x_estride = mid_stride; e2.out_estride = y_stride;
        e2.packed_problems = E; e2.packed_rt = rt_bound;
        run_big_gemm(m, "moe_gemm2", *L.e2[0], mid, o.ld4h, (long)rt_bound * 256, BEPI_F32_BIAS, e2, E);
    } else if (batched) {
        TSHIP_CHECK_HIP(hipMemcpyAsync(n_e.data(), counts, E * sizeof(int), hipMemcpyDeviceToHost, stream()));
        TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));
        for (int e = 0; e < E; ++e) TSHIP_REQUIRE(n_e[e] >= 0 && n_e[e] <= rows, "internal: expert row count out of range");
    }
    if (packed) {
        // (done above)
    } else if (m->f16 && batched) {
        half_t* xg = (half_t*)(base + o.xg); half_t* mid = (half_t*)(base + o.mid);
        launch(m, "moe_gather", moe_gather_kernel<half_t>, dim3(rows, E), dim3(256), (const float*)xn32, h, (const int*)counts, (const int*)lists, (int)Bp, xg,
               m->ldh, xg_stride, 0);
        const int n_max = *std::max_element(n_e.begin(), n_e.end());
        if (big_gemm_batched_ok(*L.e1[0], n_max) && big_gemm_batched_ok(*L.e2[0], n_max) && L.wtab1.p && L.wtab2.p && !g_hooks.no_moe_batch) {
            // all experts in one launch per projection (row counts read on the device): the down projection of one expert
            // is 64 tiles at 8 x 4096 rows, a quarter of the compute units
            BigArgs e1; std::memset(&e1, 0, sizeof(e1));
            e1.bias = zero; e1.out16 = mid; e1.ld16 = (int)o.ld4h; e1.act = c.act; e1.gated = 0; e1.n_valid = 4 * h;
            e1.Wtab = (const half_t* const*)L.wtab1.p; e1.rows_tab = counts; e1.x_estride = xg_stride; e1.out16_estride = mid_stride;
            run_big_gemm(m, "moe_gemm1", *L.e1[0], xg, m->ldh, n_max, BEPI_ACT16, e1, E);
            BigArgs e2; std::memset(&e2, 0, sizeof(e2));
            e2.bias = zero; e2.out = y; e2.ld_out = (int)o.ldy; e2.n_valid = h;
            e2.Wtab = (const half_t* const*)L.wtab2.p; e2.rows_tab = counts; e2.x_estride = mid_stride; e2.out_estride = y_stride;
            run_big_gemm(m, "moe_gemm2", *L.e2[0], mid, o.ld4h, n_max, BEPI_F32_BIAS, e2, E);
        } else {
            for (int e = 0; e < E; ++e) {
                if (n_e[e] == 0) continue;
                BigArgs e1; std::memset(&e1, 0, sizeof(e1));
                e1.bias = zero; e1.out16 = mid + e * mid_stride; e1.ld16 = (int)o.ld4h; e1.act = c.act; e1.gated = 0; e1.n_valid = 4 * h;
                run_big_gemm(m, "moe_gemm1", *L.e1[e], xg + e * xg_stride, m->ldh, n_e[e], BEPI_ACT16, e1);
                BigArgs e2; std::memset(&e2, 0, sizeof(e2));
                e2.bias = zero; e2.out = y + e * y_stride; e2.ld_out = (int)o.ldy; e2.n_valid = h;
                run_big_gemm(m, "moe_gemm2", *L.e2[e], mid + e * mid_stride, o.ld4h, n_e[e], BEPI_F32_BIAS, e2);
            }
        }
    } else if (m->f16) {
        half_t* xg = (half_t*)(base + o.xg); half_t* mid = (half_t*)(base + o.mid);
        if (fused_route) {}
        else if (fused_lists) launch(m, "moe_gather", moe_gather_lists_kernel<half_t>, dim3(rows, E), dim3(256), (const float*)top_idx, rows, k, (const float*)xn32, h,
                                counts, lists, slot, (int)Bp, xg, m->ldh, xg_stride, (int)(m->ldh / 16));
        else launch(m, "moe_gather", moe_gather_kernel<half_t>, dim3(rows, E), dim3(256), (const float*)xn32, h, (const int*)counts, (const int*)lists, (int)Bp, xg,
               m->ldh, xg_stride, (int)(m->ldh / 16));
        // (the experts' weight pointer tables were written once, when the model was finalised: no host work in a step)
        TSHIP_REQUIRE(L.wtab1.p && L.wtab2.p, "internal: expert pointer tables missing (TSHip_GptFinalize builds them)");
        SkinnyArgs e1; std::memset(&e1, 0, sizeof(e1));
        e1.W = L.e1[0]->buf.as<half_t>(); e1.KT = L.e1[0]->KT; e1.NT = L.e1[0]->NT; e1.X = xg; e1.ldx = (int)m->ldh; e1.KS = 1;
        e1.bias = zero; e1.out16 = mid; e1.ld16 = (int)o.ld4h; e1.out16_kt = L.e2[0]->KT; e1.act = c.act; e1.gated = 0; e1.n_valid = 4 * h;
        e1.Wtab = (const half_t* const*)L.wtab1.p; e1.x_estride = xg_stride; e1.out16_estride = mid_stride; e1.rows_tab = counts;
        SkinnyArgs e2; std::memset(&e2, 0, sizeof(e2));
        e2.W = L.e2[0]->buf.as<half_t>(); e2.KT = L.e2[0]->KT; e2.NT = L.e2[0]->NT; e2.X = mid; e2.ldx = (int)o.ld4h; e2.KS = 1;
        e2.bias = zero; e2.out = y; e2.ld_out = (int)o.ldy; e2.n_valid = h;
        e2.Wtab = (const half_t* const*)L.wtab2.p; e2.x_estride = mid_stride; e2.out_estride = y_stride; e2.rows_tab = counts;
        // Up projection: one 32-row tile per block with the tile number on blockIdx.z.  The experts of a decode step mostly
        // hold fewer than 32 rows, so the kernel for one row tile does the work (single-barrier reduction) and the blocks of
        // empty row tiles exit at once: 16.4 us against 24 us with two row tiles per block at 8 experts x 1024 x 4096.
        // Measured and not used: 2 or 4 column tiles per block with one copy of the activations (20 and 23 us), and the same
        // split for the down projection (19.1 against 17.9 us: its 256 blocks are one round either way).
        e1.row_tiles_z = 1;
        launch_skinny(m, "moe_gemm1", skinny_gemm_f16_kernel<1, EPI_ACT16, 8, 8, 1, false, true>, dim3(e1.NT, E, (unsigned)m->BT), dim3(512), e1);
        dim3 g2(e2.NT, E);
        if (m->BT == 1) launch_skinny(m, "moe_gemm2", skinny_gemm_f16_kernel<1, EPI_F32_BIAS, 8, 8, 1, false, true>, g2, dim3(512), e2);
        else if (m->BT == 2) launch_skinny(m, "moe_gemm2", skinny_gemm_f16_kernel<2, EPI_F32_BIAS, 8, 8, 1, false, true>, g2, dim3(512), e2);
        else launch_skinny(m, "moe_gemm2", skinny_gemm_f16_kernel<4, EPI_F32_BIAS, 4, 8, 1, false, true>, g2, dim3(256), e2);
    } else {
        float* xg = (float*)(base + o.xg); float* mid = (float*)(base + o.mid);
        if (fused_lists) launch(m, "moe_gather", moe_gather_lists_kernel<float>, dim3(rows, E), dim3(256), (const float*)top_idx, rows, k, (const float*)xn32, h,
                                counts, lists, slot, (int)Bp, xg, m->ldh, xg_stride, 0);
        else launch(m, "moe_gather", moe_gather_kernel<float>, dim3(rows, E), dim3(256), (const float*)xn32, h, (const int*)counts, (const int*)lists, (int)Bp, xg,
               m->ldh, xg_stride, 0);
        for (int e = 0; e < E; ++e) {
            // fp32 models, decode: every expert runs on `rows` rows (no host round trip for the counts); rows past the
            // expert's count hold stale finite data and are never read back.  Batched: the expert's own rows.
            const int er = n_e[e];
            if (er == 0) continue;
            float* mid_e = mid + e * mid_stride;
            run_gemm_f32(m, "moe_gemm1", *L.e1[e], xg + e * xg_stride, m->ldh, er, mid_e, o.ld4h, 0, 1);
            long tot = (long)er * 4 * h;
            launch(m, "moe_act", ffn_act_kernel<float>, dim3((unsigned)ceil_div(tot, 256)), dim3(256), (const float*)mid_e, 1, 0L, o.ld4h,
                   (const float*)zero, (const float*)zero, 4 * h, 0, (int)c.act, mid_e, o.ld4h, (long)er);
            run_gemm_f32(m, "moe_gemm2", *L.e2[e], mid_e, o.ld4h, er, y + e * y_stride, o.ldy, 0, 1);
        }
    }
    if (next) {
        ResidNormArgs a = *next;
        a.moe_y = y; a.moe_ldy = o.ldy; a.moe_estride = y_stride; a.moe_probs = probs; a.moe_top = top_idx; a.moe_slot = slot; a.moe_k = k; a.moe_E = E;
        a.moe_clear_counts = fused_route ? counts : nullptr;
        run_resid_norm(m, "moe_combine_norm", rows, a);
    } else {
        launch(m, "moe_combine", moe_combine_kernel, dim3(rows), dim3(256), pre.x, pre.ldx, h, (const float*)y, o.ldy, y_stride, (const float*)probs,
               (const float*)top_idx, (const int*)slot, k, E, fused_route ? counts : (int*)nullptr);
    }
    if (batched && last_rows) {
        // what TSHip_GptGetMoeRouting reports after a prefill: the routing of every sequence's last position
        MoeRowsArgs ra; std::memset(&ra, 0, sizeof(ra));
        ra.row_map = last_rows;
        ra.src[0] = probs; ra.dst[0] = lroute; ra.width[0] = E;
        ra.src[1] = top_val; ra.dst[1] = lroute + (size_t)m->Bpad * E; ra.width[1] = k;
        ra.src[2] = top_idx; ra.dst[2] = lroute + (size_t)m->Bpad * (E + k); ra.width[2] = k;
        launch(m, "moe_last_rows", moe_rows_kernel, dim3(n_last, 3), dim3(64), ra);
    }
}

static void run_moe_ffn(TSHipGpt* m, LayerW& L, int rows, const ResidNormArgs& pre, const ResidNormArgs* next) { run_moe_ffn_impl(m, L, rows, pre, false, m->Bpad, nullptr, 0, next); }

static void run_moe_ffn_prefill(TSHipGpt* m, LayerW& L, int rows, const ResidNormArgs& pre, const int* last_rows, int n_last, const ResidNormArgs* next) {
    const long cap = round_up(rows, 128);
    m->pw_moe.reserve(moe_layout(m, cap).total);
    run_moe_ffn_impl(m, L, rows, pre, true, cap, last_rows, n_last, next);
}

// next tokens from the logits on the device -> m->ids (and gen_out); greedy or top-p.
// With d_step set, gen_out and dev_uniforms are bases indexed by the device step counter (graph replays).
// record: the chosen tokens are about to be appended (generate loop), so their position enters the token history.
// top-p pick whose block goes on with the next decode step's first kernel for its row (as greedy_embed_kernel does)
template <int NPT>
__global__ __launch_bounds__(PICK_THREADS) void topp_pick_embed_kernel(TopPArgs a, FnPrepArgs pa) {
    const int tok = topp_pick_scan_row(a);
    fn_prepare_row<NPT, PICK_THREADS>(pa, blockIdx.x, tok, threadIdx.x);
}

// embed_next: a decode step on these tokens follows at once (the generate loop): on the fused-norm path the greedy kernel
// then also does that step's first kernel for its row and sets m->embed_done.
static void sample_tokens(TSHipGpt* m, int mode, float top_p, float temperature, const float* host_uniforms, const float* dev_uniforms, int B,
                          int* gen_out, const int* d_step, bool record, bool embed_next) {
    const long Vp = round_up(m->c.vocab, 32);
    int* last = m->last_pos.as<int>();           // null unless a repeat penalty was set
    if (last) TSHIP_REQUIRE((size_t)B * m->last_ld * sizeof(int) <= m->last_pos.bytes && m->last_ld >= m->c.vocab, "internal: token history table too small");
    if (mode == TSHIP_GREEDY) {
        const float* lg = m->logits.as<float>(); int* ids = m->ids.as<int>(); int* lastp = record ? last : (int*)nullptr;
        const int* dpos = m->d_pos.as<int>(); const unsigned char* bl = m->any_blocked ? (const unsigned char*)m->blocked.p : (const unsigned char*)nullptr;
        if (embed_next && m->fused_norm && m->c.hidden <= 8192) {
            const FnPrepArgs pa = embed_prepare_args(m, ids);
            const int h = m->c.hidden;
            if (h <= 2048) launch(m, "greedy_embed", greedy_embed_kernel<2>, dim3(B), dim3(1024), lg, Vp, m->c.vocab, ids, gen_out, d_step, lastp, m->last_ld, dpos, bl, pa);
            else if (h <= 4096) launch(m, "greedy_embed", greedy_embed_kernel<4>, dim3(B), dim3(1024), lg, Vp, m->c.vocab, ids, gen_out, d_step, lastp, m->last_ld, dpos, bl, pa);
            else launch(m, "greedy_embed", greedy_embed_kernel<8>, dim3(B), dim3(1024), lg, Vp, m->c.vocab, ids, gen_out, d_step, lastp, m->last_ld, dpos, bl, pa);
            m->embed_done = true;
            return;
        }
        launch(m, "greedy", greedy_kernel, dim3(B), dim3(1024), lg, Vp, m->c.vocab, ids, gen_out, d_step, lastp, m->last_ld, dpos, bl);
        return;
    }
    TSHIP_REQUIRE(mode == TSHIP_TOPP, "unknown sampling mode");
    TSHIP_REQUIRE(m->c.vocab <= 262144, "top-p sampling supports vocabularies up to 262144");
    TSHIP_REQUIRE(temperature > 0.0f, "temperature must be positive");
    const size_t need = topp_scratch_bytes(m->Bpad, m->c.vocab);
    if (m->topp_scratch.bytes < need) m->topp_scratch.alloc(need);
    if (!dev_uniforms) {
        TSHIP_REQUIRE(host_uniforms, "top-p sampling needs one uniform draw per row");
        if (m->topp_uni.bytes < (size_t)m->Bpad * 4) m->topp_uni.alloc((size_t)m->Bpad * 4);
        TSHIP_CHECK_HIP(hipMemcpyAsync(m->topp_uni.p, host_uniforms, (size_t)B * 4, hipMemcpyHostToDevice, stream()));
        dev_uniforms = m->topp_uni.as<float>();
    }
    TopPArgs a; std::memset(&a, 0, sizeof(a));
    a.in = m->logits.as<float>(); a.ld = Vp; a.V = m->c.vocab; a.in_is_logits = 1;
    a.uniforms = dev_uniforms; a.top_p = top_p;
    topp_carve(a, m->topp_scratch.p, m->Bpad, m->c.vocab);
    a.next_ids = m->ids.as<int>(); a.gen_out = gen_out; a.d_step = d_step;
    // Decoder.cs:720-723 divides the logits by the temperature (fp32 division) before the softmax
    a.temperature = temperature;
    // Decoder.cs:761: TopPSample(probs, TopP, RepeatPenalty, decodedSequences: tgtSeqs); the sequence length is the number
    // of cached positions
    a.blocked = m->any_blocked ? (const unsigned char*)m->blocked.p : nullptr;
    a.repeat_penalty = m->repeat_penalty; a.last_pos = last; a.last_ld = m->last_ld; a.d_len = m->d_pos.as<int>(); a.record = record ? 1 : 0;
    auto run = [&](const char* name, void (*kernel)(TopPArgs), dim3 grid, dim3 block, const TopPArgs& args) { launch(m, name, kernel, grid, block, args); };
    if (embed_next && m->fused_norm && m->c.hidden <= 8192) {
        const TopPArgs pick = topp_run(a, B, run, false);
        const FnPrepArgs pa = embed_prepare_args(m, m->ids.as<int>());
        const int h = m->c.hidden;
        if (h <= 2048) launch(m, "topp_pick_embed", topp_pick_embed_kernel<4>, dim3(B), dim3(PICK_THREADS), pick, pa);
        else if (h <= 4096) launch(m, "topp_pick_embed", topp_pick_embed_kernel<8>, dim3(B), dim3(PICK_THREADS), pick, pa);
        else launch(m, "topp_pick_embed", topp_pick_embed_kernel<16>, dim3(B), dim3(PICK_THREADS), pick, pa);
        m->embed_done = true;
        return;
    }
    topp_run(a, B, run);
}

}  // namespace tship
